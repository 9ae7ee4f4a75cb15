"""Host mirror of jitnn-llm's Llm (jitnn-llm/src/main/java/ai/beestream/jitnn/llm/Llm.java:48-120): a GGUF language model
that generates text.  The reference hands generation to the third-party jitllm engine; here the file's quantised weights
are attached to the decode step of libjitnn_hip.so (jitnn_hip_llama_*), the token loop runs in the library
(jitnn_hip_llama_generate: embedding lookup, prompt pass, greedy choice, token-by-token decode over the KV cache) and the
tokenizer is built from the file's metadata (tokenizer.py).

    with Llm.load("model.gguf") as llm:
        answer = llm.generate("What is the capital of France?", 64)
        result = llm.generate(GenerationRequest("Once upon a time", 200, temperature=0.8, top_p=0.95, seed=1, stop=["\n\n"]))

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


class GenerationRequest:
    """What Llm.generate(request) hands to the engine (Llm.java:84-93 passes a jitllm GenerationRequest through): the prompt,
    the length limit, sampling and stop sequences.  temperature 0 is the greedy choice; top_k 0 and top_p 1 put no limit
    on the candidates; seed None draws from a fresh generator.  Chat messages and tools are jitllm's and are not built."""

    def __init__(self, prompt: str, max_new_tokens: int = 128, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed=None,
                 stop=(), on_token=None):
        if max_new_tokens < 0 or temperature < 0 or top_k < 0 or not 0.0 < top_p <= 1.0:
            raise ValueError(f"max_new_tokens {max_new_tokens}, temperature {temperature}, top_k {top_k}, top_p {top_p}")
        self.prompt, self.max_new_tokens, self.temperature, self.top_k, self.top_p = prompt, max_new_tokens, float(temperature), int(top_k), float(top_p)
        self.seed, self.stop, self.on_token = seed, tuple(s for s in ([stop] if isinstance(stop, str) else stop) if s), on_token


class GenerationResult:
    """text: the continuation (cut in front of the stop sequence that ended it); tokens: the ids that were produced;
    finish_reason: "eos" (the model's end-of-sequence token), "stop" (a stop sequence) or "length"."""

    def __init__(self, text, tokens, prompt_tokens, finish_reason):
        self.text, self.tokens, self.prompt_tokens, self.finish_reason = text, tokens, prompt_tokens, finish_reason

    def __repr__(self):
        return f"GenerationResult({self.text!r}, {len(self.tokens)} tokens after {self.prompt_tokens}, {self.finish_reason})"


def sample_token(logits, temperature: float, top_k: int, top_p: float, rng) -> int:
    """One token id from logits [vocab].  temperature 0: the largest logit, the lowest index among equals, NaN never (what
    the device kernel of the greedy loop picks).  Otherwise softmax(logits / temperature) over the top_k largest (0: all),
    cut to the smallest set of most likely tokens whose probability reaches top_p, renormalised, and one draw of rng."""
    a = np.asarray(logits, dtype=np.float64).reshape(-1)
    a = np.where(np.isnan(a), -np.inf, a)
    if temperature <= 0.0 or top_k == 1:
        return int(np.argmax(a))
    order = np.argsort(-a, kind="stable")  # most likely first, the lower index first among equals
    if top_k > 0:
        order = order[:top_k]
    z = a[order] / temperature
    z -= z[0]
    p = np.exp(z)
    p /= p.sum()
    if top_p < 1.0:
        keep = int(np.searchsorted(np.cumsum(p), top_p, side="left")) + 1
        order, p = order[:keep], p[:keep] / p[:keep].sum()
    return int(order[min(int(np.searchsorted(np.cumsum(p), rng.random(), side="right")), len(order) - 1)])


class StopFilter:
    """Text pieces in, text pieces out, holding back whatever could still turn into a stop sequence: push returns
    (text to emit, stopped); after a stop nothing more comes out and the stop sequence itself is never emitted."""

    def __init__(self, stop):
        self._stop, self._held, self.stopped = tuple(stop), "", False

    def push(self, piece: str):
        if self.stopped:
            return "", True
        text = self._held + piece
        cut = min((i for i in (text.find(s) for s in self._stop) if i >= 0), default=-1)
        if cut >= 0:
            self._held, self.stopped = "", True
            return text[:cut], True
        hold = 0
        for s in self._stop:  # the longest tail of the text that begins a stop sequence stays back
            for n in range(min(len(s) - 1, len(text)), 0, -1):
                if text.endswith(s[:n]):
                    hold = max(hold, n)
                    break
        self._held = text[len(text) - hold:] if hold else ""
        return text[:len(text) - hold] if hold else text, False

    def flush(self) -> str:
        out, self._held = ("" if self.stopped else self._held), ""
        return out


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

    def generate(self, prompt, max_new_tokens: int | None = None, on_text=None):
        """generate(prompt, max_new_tokens[, on_text]): the greedy (temperature 0) continuation of `prompt` as a string, at most
        `max_new_tokens` tokens, each piece of text going to `on_text` as it is produced (Llm.generate, Llm.java:74-82).
        generate(request): a GenerationRequest - sampling, stop sequences - to a GenerationResult (Llm.java:84-93)."""
        if isinstance(prompt, GenerationRequest):
            return self._generate_request(prompt)
        if max_new_tokens is None:
            raise TypeError("generate(prompt, max_new_tokens) or generate(GenerationRequest)")
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

    def _generate_request(self, rq: GenerationRequest) -> GenerationResult:
        """The token loop on the host, for requests the library's greedy loop does not cover: the prompt in one pass
        (jitnn_hip_llama_prefill), then logits -> sample_token -> embedding row -> one decode step per token."""
        ids = self._tok.encode(rq.prompt)
        if not ids:
            raise ValueError("the prompt has no tokens")
        if len(ids) + rq.max_new_tokens > self._info.context:
            raise ValueError(f"{len(ids)} prompt tokens + {rq.max_new_tokens} new ones in a context of {self._info.context}")
        eos = self._tok.eos if self._tok.eos is not None else -1
        rng = np.random.default_rng(rq.seed)
        stream, stops = StreamDecoder(self._tok), StopFilter(rq.stop)
        pieces, out, reason = [], [], "length"

        def emit(s):
            s, stopped = stops.push(s)
            if s:
                pieces.append(s)
                if rq.on_token is not None:
                    rq.on_token(s)
            return stopped

        if rq.max_new_tokens > 0:
            logits = self._dec.prefill(self._dec.embed(ids), 0)
            pos = len(ids)
            while True:
                token = sample_token(logits, rq.temperature, rq.top_k, rq.top_p, rng)
                if token == eos:
                    reason = "eos"
                    break
                out.append(token)
                if emit(stream.push(token)):
                    reason = "stop"
                    break
                if len(out) == rq.max_new_tokens:
                    break
                logits = self._dec.decode(self._dec.embed([token])[0], pos)
                pos += 1
        if reason != "stop":
            if emit(stream.flush()):
                reason = "stop"
            tail = stops.flush()
            if tail:
                pieces.append(tail)
                if rq.on_token is not None:
                    rq.on_token(tail)
        return GenerationResult("".join(pieces), out, len(ids), reason)

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
