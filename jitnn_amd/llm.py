"""Host mirror of jitnn-llm's Llm (jitnn-llm/src/main/java/ai/beestream/jitnn/llm/Llm.java:48-139): a GGUF language model
that generates text.  The reference hands generation to the third-party jitllm engine; here the file's quantised weights
are attached to the decode step of libjitnn_hip.so (jitnn_hip_llama_*), the token loop runs in the library
(jitnn_hip_llama_generate: embedding lookup, prompt pass, greedy choice, token-by-token decode over the KV cache) and the
tokenizer is built from the file's metadata (tokenizer.py).

    with Llm.load("model.gguf") as llm:
        answer = llm.generate("What is the capital of France?", 64)

Llama-style architectures only (RMSNorm, rotary embedding, grouped-query attention, SwiGLU: general.architecture "llama",
and the same tensor layout under other names where the metadata says so); anything else raises.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .gguf_file import GgufFile
from .llama import LlamaDecoder, W_OUTPUT
from .tokenizer import StreamDecoder, Tokenizer

# GGUF tensor names of a Llama-style layer in the order of the decoder's weight slots
LAYER_TENSORS = ["attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"]
INTERLEAVED_ROPE_ARCHS = {"llama", "mistral", "granite"}  # llama.cpp's "NORM" rotary embedding: q and k stored permuted for pairs (2i, 2i + 1)

_TOKEN_CB = C.CFUNCTYPE(None, C.c_int, C.c_void_p)


class ModelInfo:
    def __init__(self, architecture, name, layers, d_model, heads, kv_heads, head_dim, ffn, vocab, context, quantisation):
        self.architecture, self.name, self.layers, self.d_model, self.heads, self.kv_heads = architecture, name, layers, d_model, heads, kv_heads
        self.head_dim, self.ffn, self.vocab, self.context, self.quantisation = head_dim, ffn, vocab, context, quantisation

    def __repr__(self):
        return (f"ModelInfo({self.architecture} {self.name!r}: {self.layers} layers, d_model {self.d_model}, {self.heads}/{self.kv_heads} heads of "
                f"{self.head_dim}, ffn {self.ffn}, vocab {self.vocab}, context {self.context}, weights {self.quantisation})")


class Llm:
    def __init__(self, gguf: GgufFile, decoder: LlamaDecoder, tokenizer: Tokenizer, info: ModelInfo):
        self._gguf, self._dec, self._tok, self._info = gguf, decoder, tokenizer, info

    @staticmethod
    def load(path, max_context: int | None = None) -> "Llm":
        """Opens the file, uploads its weights (raw blocks, unchanged) and builds the tokenizer (Llm.load, Llm.java:58-72)."""
        f = GgufFile.open(path)
        try:
            arch = f.architecture()
            if arch is None:
                raise ValueError(f"{path}: no general.architecture")
            layers = f.integer(f"{arch}.block_count")
            d = f.integer(f"{arch}.embedding_length")
            heads = f.integer(f"{arch}.attention.head_count")
            kv = f.integer(f"{arch}.attention.head_count_kv", heads)
            ffn = f.integer(f"{arch}.feed_forward_length")
            hd = f.integer(f"{arch}.attention.key_length", d // heads)
            eps = f.float_value(f"{arch}.attention.layer_norm_rms_epsilon", 1e-5)
            theta = f.float_value(f"{arch}.rope.freq_base", 10000.0)
            ctx_file = f.integer(f"{arch}.context_length", 2048)
            for name in ("token_embd.weight", "output_norm.weight", "blk.0.attn_q.weight", "blk.0.ffn_gate.weight"):
                if not f.has_tensor(name):
                    raise ValueError(f"{path}: architecture {arch} does not generate text here (no tensor {name}; Llama-style layers are built)")
            emb = f.info("token_embd.weight")
            vocab = emb.shape[0]
            ctx = min(ctx_file, max_context) if max_context else min(ctx_file, 4096)
            dec = LlamaDecoder(layers, d, heads, kv, hd, ffn, vocab, ctx, eps, theta)
            fmts = set()
            for l in range(layers):
                for slot, tn in enumerate(LAYER_TENSORS):
                    w = f.tensor(f"blk.{l}.{tn}.weight")
                    fmts.add(w.dtype().name)
                    dec.set_weight(l, slot, w)
                dec.set_norm(l, 0, f.raw(f"blk.{l}.attn_norm.weight").view(np.float32))
                dec.set_norm(l, 1, f.raw(f"blk.{l}.ffn_norm.weight").view(np.float32))
            dec.set_norm(0, 2, f.raw("output_norm.weight").view(np.float32))
            # the output head; files with tied embeddings have none and use the token table
            dec.set_weight(0, W_OUTPUT, f.tensor("output.weight" if f.has_tensor("output.weight") else "token_embd.weight"))
            dec.set_embedding(emb.type_id, f.raw("token_embd.weight"))
            dec.set_rope_interleaved(arch in INTERLEAVED_ROPE_ARCHS)
            tok = Tokenizer.from_gguf(f)
            if len(tok.tokens) != vocab:
                raise ValueError(f"{path}: {len(tok.tokens)} tokens for an embedding table of {vocab} rows")
            name = f.get("general.name") if f.has("general.name") else ""
            info = ModelInfo(arch, name, layers, d, heads, kv, hd, ffn, vocab, ctx, "+".join(sorted(fmts)))
            return Llm(f, dec, tok, info)
        except Exception:
            f.close()
            raise

    def generate(self, prompt: str, max_new_tokens: int, on_text=None) -> str:
        """The greedy (temperature 0) continuation of `prompt`, at most `max_new_tokens` tokens; each piece of text goes to
        `on_text` as it is produced (Llm.generate, Llm.java:74-82)."""
        ids = self._tok.encode(prompt)
        if not ids:
            raise ValueError("the prompt has no tokens")
        stream = StreamDecoder(self._tok)
        pieces = []

        def on_token(token, _user):
            s = stream.push(token)
            if s:
                pieces.append(s)
                if on_text is not None:
                    on_text(s)

        self.generate_tokens(ids, max_new_tokens, on_token)
        tail = stream.flush()
        if tail:
            pieces.append(tail)
            if on_text is not None:
                on_text(tail)
        return "".join(pieces)

    def generate_tokens(self, prompt_ids, max_new_tokens: int, on_token=None, pos0: int = 0) -> list:
        """Token ids in, token ids out: the loop of jitnn_hip_llama_generate (stops at the file's end-of-sequence token)."""
        eos = self._tok.eos if self._tok.eos is not None else -1
        return self._dec.generate(prompt_ids, max_new_tokens, eos, on_token, pos0)

    def gguf(self) -> GgufFile:
        return self._gguf

    def tokenizer(self) -> Tokenizer:
        return self._tok

    def model(self) -> LlamaDecoder:
        return self._dec

    def info(self) -> ModelInfo:
        return self._info

    def close(self):
        self._dec.close()
        self._gguf.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False
