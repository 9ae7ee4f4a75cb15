"""The decode step composed from the CPU oracle's operators, in the order of the reference's Llama.Block.forward
(jitnn-nn/src/main/java/ai/beestream/jitnn/nn/models/Llama.java:167-174,209-222) with every Linear replaced by
Gguf.linear on raw blocks and the one new token attending an FP32 cache.  Test infrastructure."""
from __future__ import annotations

import numpy as np

from oracle import oracle

SLOTS = ["attn_q", "attn_k", "attn_v", "attn_o", "ffn_gate", "ffn_up", "ffn_down"]


def decode_ref(cfg, layers, out_norm, out_w, kcache, vcache, x, pos):
    """layers: list of dicts {slot: (ggml id, raw, n, k)} + 'attn_norm', 'ffn_norm'; out_w = (id, raw, n, k);
    kcache/vcache [L, ctx, kv, hd] are updated in place at pos.  Returns logits [vocab]."""
    heads, kv, hd = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_eps"], np.float32(cfg["rope_theta"])

    def lin(w, a):
        fid, raw, n, k = w
        return oracle.gguf_linear(fid, a.reshape(1, k), raw, None, n, k)[0]

    x = np.asarray(x, dtype=np.float32)
    for li, L in enumerate(layers):
        n = oracle.rms_norm(x, L["attn_norm"], eps)
        q = oracle.rope(lin(L["attn_q"], n).reshape(1, heads, hd), theta, pos, False, True)[0]
        k = oracle.rope(lin(L["attn_k"], n).reshape(1, kv, hd), theta, pos, False, True)[0]
        v = lin(L["attn_v"], n).reshape(kv, hd)
        kcache[li, pos], vcache[li, pos] = k, v
        att = oracle.attention_decode(q, kcache[li, :pos + 1], vcache[li, :pos + 1])
        x = oracle.add(x, lin(L["attn_o"], att.reshape(-1)))
        m = oracle.rms_norm(x, L["ffn_norm"], eps)
        x = oracle.add(x, lin(L["ffn_down"], oracle.swiglu(lin(L["ffn_gate"], m), lin(L["ffn_up"], m))))
    return lin(out_w, oracle.rms_norm(x, out_norm, eps))
