"""Host mirror of the decode-step entry points (jitnn_hip_llama_*): a Llama-style stack whose linears are
quantised weights, one token per step over an FP32 KV cache.  The arithmetic is the reference's Llama.Block.forward
(jitnn-nn/src/main/java/ai/beestream/jitnn/nn/models/Llama.java:167-174,209-222) with Gguf.linear in place of Linear."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .tensor import Tensor

W_ATTN_Q, W_ATTN_K, W_ATTN_V, W_ATTN_O, W_FFN_GATE, W_FFN_UP, W_FFN_DOWN, W_OUTPUT = range(8)
NORM_ATTN, NORM_FFN, NORM_OUTPUT = range(3)


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class LlamaDecoder:
    def __init__(self, layers, d_model, heads, kv_heads, head_dim, ffn, vocab, max_ctx, rms_eps=1e-5, rope_theta=5e5):
        _lib.init()
        self.cfg = dict(layers=layers, d_model=d_model, heads=heads, kv_heads=kv_heads, head_dim=head_dim, ffn=ffn, vocab=vocab,
                        max_ctx=max_ctx, rms_eps=rms_eps, rope_theta=rope_theta)
        self._h = C.c_void_p()
        _lib.check(_lib.lib.jitnn_hip_llama_create(layers, d_model, heads, kv_heads, head_dim, ffn, vocab, max_ctx, rms_eps, rope_theta,
                                                   C.byref(self._h)), "jitnn_hip_llama_create")
        self._keep = []  # weights are not owned by the native model: keep their tensors alive

    def close(self):
        if self._h:
            _lib.lib.jitnn_hip_llama_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self):
        return self._h

    def set_weight(self, layer: int, which: int, w: Tensor) -> None:
        _lib.check(_lib.lib.jitnn_hip_llama_set_weight(self._h, layer, which, w.handle), "jitnn_hip_llama_set_weight")
        self._keep.append(w)

    def set_weight_handle(self, layer: int, which: int, handle) -> None:
        _lib.check(_lib.lib.jitnn_hip_llama_set_weight(self._h, layer, which, handle), "jitnn_hip_llama_set_weight")

    def set_norm(self, layer: int, which: int, w) -> None:
        a = np.ascontiguousarray(w, dtype=np.float32)
        if a.size != self.cfg["d_model"]:
            raise ValueError(f"norm weight of {a.size} values for d_model {self.cfg['d_model']}")
        _lib.check(_lib.lib.jitnn_hip_llama_set_norm(self._h, layer, which, _p(a)), "jitnn_hip_llama_set_norm")

    def kv_write(self, layer: int, pos0: int, k, v) -> None:
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        row = self.cfg["kv_heads"] * self.cfg["head_dim"]
        if k.shape != v.shape or k.size % row != 0:
            raise ValueError(f"cache rows of shape {k.shape} / {v.shape}")
        _lib.check(_lib.lib.jitnn_hip_llama_kv_write(self._h, layer, pos0, k.size // row, _p(k), _p(v)), "jitnn_hip_llama_kv_write")

    def kv_read(self, layer: int, pos0: int, count: int):
        shape = (count, self.cfg["kv_heads"], self.cfg["head_dim"])
        k, v = np.empty(shape, dtype=np.float32), np.empty(shape, dtype=np.float32)
        _lib.check(_lib.lib.jitnn_hip_llama_kv_read(self._h, layer, pos0, count, _p(k), _p(v)), "jitnn_hip_llama_kv_read")
        return k, v

    def decode(self, x, pos: int) -> np.ndarray:
        """Logits [vocab] of the token whose embedding is x [d_model] at position pos."""
        a = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
        if a.size != self.cfg["d_model"]:
            raise ValueError(f"embedding of {a.size} values for d_model {self.cfg['d_model']}")
        y = np.empty(self.cfg["vocab"], dtype=np.float32)
        _lib.check(_lib.lib.jitnn_hip_llama_decode(self._h, _p(a), pos, _p(y)), "jitnn_hip_llama_decode")
        return y

    def decode_dev(self, x_ptr: int, pos: int, logits_ptr: int, stream_ptr: int = 0) -> None:
        _lib.check(_lib.lib.jitnn_hip_llama_decode_dev(self._h, C.c_void_p(x_ptr), pos, C.c_void_p(logits_ptr), C.c_void_p(stream_ptr)),
                   "jitnn_hip_llama_decode_dev")

    def set_rope_interleaved(self, on: bool) -> None:
        """Rotary pairs (2i, 2i + 1) instead of the default (i, i + head_dim / 2): the two forms of Rope (core/ops/Rope.java:126-150)."""
        _lib.check(_lib.lib.jitnn_hip_llama_set_rope_interleaved(self._h, 1 if on else 0), "jitnn_hip_llama_set_rope_interleaved")

    def set_embedding(self, ggml_type: int, table) -> None:
        """The token embedding table [vocab, d_model] as raw bytes of ggml type F32 (0), F16 (1) or a block format."""
        raw = np.ascontiguousarray(table).view(np.uint8).reshape(-1)
        _lib.check(_lib.lib.jitnn_hip_llama_set_embedding(self._h, ggml_type, _p(raw), raw.size), "jitnn_hip_llama_set_embedding")

    def embed(self, tokens) -> np.ndarray:
        """Embedding rows [count, d_model] of token ids (through device memory; for tests)."""
        ids = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
        if ids.size and (ids.min() < 0 or ids.max() >= self.cfg["vocab"]):
            raise ValueError(f"token id outside [0, {self.cfg['vocab']})")
        n, d = ids.size, self.cfg["d_model"]
        dev_ids, dev_x = C.c_void_p(), C.c_void_p()
        _lib.check(_lib.lib.jitnn_hip_malloc(ids.nbytes, C.byref(dev_ids)), "jitnn_hip_malloc")
        _lib.check(_lib.lib.jitnn_hip_malloc(n * d * 4, C.byref(dev_x)), "jitnn_hip_malloc")
        try:
            _lib.check(_lib.lib.jitnn_hip_memcpy_h2d(dev_ids, _p(ids), ids.nbytes), "jitnn_hip_memcpy_h2d")
            _lib.check(_lib.lib.jitnn_hip_llama_embed_dev(self._h, dev_ids, n, dev_x, None), "jitnn_hip_llama_embed_dev")
            x = np.empty((n, d), dtype=np.float32)
            _lib.check(_lib.lib.jitnn_hip_memcpy_d2h(_p(x), dev_x, x.nbytes), "jitnn_hip_memcpy_d2h")
            return x
        finally:
            _lib.lib.jitnn_hip_free(dev_ids)
            _lib.lib.jitnn_hip_free(dev_x)

    def argmax(self, logits) -> int:
        """Index of the largest logit as the device kernel of the generation loop picks it (for tests)."""
        a = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
        if a.size != self.cfg["vocab"]:
            raise ValueError(f"{a.size} logits for a vocabulary of {self.cfg['vocab']}")
        dev_l, dev_t = C.c_void_p(), C.c_void_p()
        _lib.check(_lib.lib.jitnn_hip_malloc(a.nbytes, C.byref(dev_l)), "jitnn_hip_malloc")
        _lib.check(_lib.lib.jitnn_hip_malloc(4, C.byref(dev_t)), "jitnn_hip_malloc")
        try:
            _lib.check(_lib.lib.jitnn_hip_memcpy_h2d(dev_l, _p(a), a.nbytes), "jitnn_hip_memcpy_h2d")
            _lib.check(_lib.lib.jitnn_hip_llama_argmax_dev(self._h, dev_l, dev_t, None), "jitnn_hip_llama_argmax_dev")
            t = np.empty(1, dtype=np.int32)
            _lib.check(_lib.lib.jitnn_hip_memcpy_d2h(_p(t), dev_t, 4), "jitnn_hip_memcpy_d2h")
            return int(t[0])
        finally:
            _lib.lib.jitnn_hip_free(dev_l)
            _lib.lib.jitnn_hip_free(dev_t)

    def generate(self, prompt_ids, max_new_tokens: int, eos_token: int = -1, on_token=None, pos0: int = 0) -> list:
        """Greedy continuation of the prompt's token ids (jitnn_hip_llama_generate); on_token(token, None) is called for every
        new token as soon as it exists."""
        ids = np.ascontiguousarray(prompt_ids, dtype=np.int32).reshape(-1)
        out = np.empty(max(max_new_tokens, 1), dtype=np.int32)
        cb_type = C.CFUNCTYPE(None, C.c_int, C.c_void_p)
        cb = cb_type(on_token) if on_token is not None else None
        n = _lib.lib.jitnn_hip_llama_generate(self._h, _p(ids), ids.size, pos0, max_new_tokens, eos_token, _p(out),
                                              C.cast(cb, C.c_void_p) if cb is not None else None, None)
        if n < 0:
            _lib.check(n, "jitnn_hip_llama_generate")
        return [int(t) for t in out[:n]]

    def prefill(self, x, pos0: int = 0, logits: bool = True):
        """Runs the tokens whose embeddings are the rows of x [tokens, d_model] through the stack at positions
        pos0 .. pos0 + tokens - 1 (causal attention over the cache and one another), appends their keys and values,
        and returns the logits [vocab] of the last token (None when logits is False)."""
        a = np.ascontiguousarray(x, dtype=np.float32)
        if a.ndim != 2 or a.shape[1] != self.cfg["d_model"]:
            raise ValueError(f"embeddings of shape {a.shape} for d_model {self.cfg['d_model']}")
        y = np.empty(self.cfg["vocab"], dtype=np.float32) if logits else None
        _lib.check(_lib.lib.jitnn_hip_llama_prefill(self._h, _p(a), pos0, a.shape[0], _p(y) if logits else None), "jitnn_hip_llama_prefill")
        return y

    def prefill_dev(self, x_ptr: int, pos0: int, tokens: int, logits_ptr: int = 0, stream_ptr: int = 0) -> None:
        _lib.check(_lib.lib.jitnn_hip_llama_prefill_dev(self._h, C.c_void_p(x_ptr), pos0, tokens, C.c_void_p(logits_ptr), C.c_void_p(stream_ptr)),
                   "jitnn_hip_llama_prefill_dev")
