"""The decode step composed from the CPU oracle's operators, in the order of the reference's Llama.Block.forward
(jitnn-nn/src/main/java/ai/beestream/jitnn/nn/models/Llama.java:167-174,209-222) with every Linear replaced by
Gguf.linear on raw blocks and the one new token attending an FP32 cache.  Test infrastructure."""
from __future__ import annotations

import numpy as np

from oracle import oracle

SLOTS = ["attn_q", "attn_k", "attn_v", "attn_o", "ffn_gate", "ffn_up", "ffn_down"]


def decode_ref(cfg, layers, out_norm, out_w, kcache, vcache, x, pos, threads: int = 1, rope_interleaved: bool = False):
    """layers: list of dicts {slot: (ggml id, raw, n, k)} + 'attn_norm', 'ffn_norm'; out_w = (id, raw, n, k);
    kcache/vcache [L, ctx, kv, hd] are updated in place at pos.  Returns logits [vocab].
    threads > 1 shares the output rows of every linear out over host threads (bit-identical results); rope_interleaved
    selects Rope's pairs (2i, 2i + 1) instead of (i, i + D/2) (ops/Rope.java:126-150)."""
    heads, kv, hd = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_eps"], np.float32(cfg["rope_theta"])

    def lin(w, a):
        fid, raw, n, k = w
        if threads > 1 and n >= 4 * threads:
            return oracle.gguf_linear_rows_parallel(fid, a.reshape(1, k), raw, None, n, k, threads)[0]
        return oracle.gguf_linear(fid, a.reshape(1, k), raw, None, n, k)[0]

    x = np.asarray(x, dtype=np.float32)
    for li, L in enumerate(layers):
        n = oracle.rms_norm(x, L["attn_norm"], eps)
        q = oracle.rope(lin(L["attn_q"], n).reshape(1, heads, hd), theta, pos, rope_interleaved, True)[0]
        k = oracle.rope(lin(L["attn_k"], n).reshape(1, kv, hd), theta, pos, rope_interleaved, True)[0]
        v = lin(L["attn_v"], n).reshape(kv, hd)
        kcache[li, pos], vcache[li, pos] = k, v
        att = oracle.attention_decode(q, kcache[li, :pos + 1], vcache[li, :pos + 1])
        x = oracle.add(x, lin(L["attn_o"], att.reshape(-1)))
        m = oracle.rms_norm(x, L["ffn_norm"], eps)
        x = oracle.add(x, lin(L["ffn_down"], oracle.swiglu(lin(L["ffn_gate"], m), lin(L["ffn_up"], m))))
        if threads > 1 and li % 8 == 7:
            print(f"  oracle: layer {li + 1} of {len(layers)}", flush=True)
    return lin(out_w, oracle.rms_norm(x, out_norm, eps))


def prefill_ref(cfg, layers, out_norm, out_w, kcache, vcache, x, pos0):
    """The same stack on T tokens at positions pos0 .. pos0 + T - 1, layer by layer, every token exactly as decode_ref
    would treat it (token t attends positions 0 .. pos0 + t).  The linears are taken as FP64 products with the oracle's
    dequantised weights (bit-exact against the reference's fixtures) rounded to FP32 - the definition of
    Gguf.MatVec.reference (core/ops/Gguf.java:187-205) up to the summation order of the FP64 accumulator, 1e-16
    relative - so that 512 tokens do not take 512 scalar passes over every weight.
    Returns (logits of the last token [vocab], per-layer hidden states are not kept); the caches are updated in place."""
    heads, kv, hd = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_eps"], np.float32(cfg["rope_theta"])

    def lin(w, a):
        fid, raw, n, k = w
        wd = oracle.dequantize(fid, raw, n * k).reshape(n, k).astype(np.float64)
        return (a.astype(np.float64) @ wd.T).astype(np.float32)

    x = np.ascontiguousarray(x, dtype=np.float32)
    T = x.shape[0]
    for li, L in enumerate(layers):
        n = oracle.rms_norm(x, L["attn_norm"], eps)
        q = oracle.rope(lin(L["attn_q"], n).reshape(T, heads, hd), theta, pos0, False, True)
        k = oracle.rope(lin(L["attn_k"], n).reshape(T, kv, hd), theta, pos0, False, True)
        v = lin(L["attn_v"], n).reshape(T, kv, hd)
        kcache[li, pos0:pos0 + T], vcache[li, pos0:pos0 + T] = k, v
        att = np.empty((T, heads * hd), dtype=np.float32)
        for t in range(T):
            att[t] = oracle.attention_decode(q[t], kcache[li, :pos0 + t + 1], vcache[li, :pos0 + t + 1]).reshape(-1)
        x = oracle.add(x, lin(L["attn_o"], att))
        m = oracle.rms_norm(x, L["ffn_norm"], eps)
        x = oracle.add(x, lin(L["ffn_down"], oracle.swiglu(lin(L["ffn_gate"], m), lin(L["ffn_up"], m))))
    last = oracle.rms_norm(x[T - 1], out_norm, eps)
    fid, raw, n, k = out_w
    return oracle.gguf_linear_rows_parallel(fid, last.reshape(1, k), raw, None, n, k, 8)[0]
