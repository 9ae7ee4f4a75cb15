"""Pins the decode-step glue oracle (oracle/jitnn_glue_oracle.c) against the reference's goldens."""
import numpy as np

from helpers import checks_close
from oracle import oracle

RT, AT = 1e-4, 1e-4  # Golden.java:483-498 (accumulating ops)


def test_rms_norm(goldens):
    for name in ("rms_norm", "rms_norm_3d", "rms_norm_long", "rms_norm_rows"):
        c = goldens[name]
        y = oracle.rms_norm(c.arrays["in0"], c.arrays["in1"], float(c.attrs[0]))
        assert checks_close(y, c.arrays["out"], RT, AT), name
        assert np.abs(y - c.arrays["out"]).max() <= 1e-6 * max(1.0, np.abs(c.arrays["out"]).max())


def test_rope(goldens):
    for name, heads in (("rope_heads", True), ("rope_heads_interleaved", True), ("rope_half", False), ("rope_offset", False),
                        ("rope_long", False)):
        c = goldens[name]
        base, offset, inter = float(c.attrs[0]), int(c.attrs[1]), bool(int(c.attrs[2]))
        y = oracle.rope(c.arrays["in0"], np.float32(base), offset, inter, heads)
        assert checks_close(y, c.arrays["out"], RT, AT), name
        assert np.abs(y - c.arrays["out"]).max() <= 2e-5, name


def test_silu_swiglu(goldens):
    for name in ("silu", "silu_tails"):
        c = goldens[name]
        assert checks_close(oracle.silu(c.arrays["in0"]), c.arrays["out"], 1e-5, 1e-6), name
    c = goldens["swiglu"]
    assert checks_close(oracle.swiglu(c.arrays["in0"], c.arrays["in1"]), c.arrays["out"], 1e-5, 1e-6)


def test_sdpa(goldens):
    for name in ("sdpa", "sdpa_causal", "sdpa_head128"):
        c = goldens[name]
        y = oracle.sdpa(c.arrays["in0"], c.arrays["in1"], c.arrays["in2"], bool(int(c.attrs[0])), float(c.attrs[1]))
        assert checks_close(y, c.arrays["out"], RT, AT), name
    c = goldens["sdpa_bthd_causal"]  # [B, T, H, E]
    q, k, v = (np.ascontiguousarray(c.arrays[n].transpose(0, 2, 1, 3)) for n in ("in0", "in1", "in2"))
    y = oracle.sdpa(q, k, v, True, -1).transpose(0, 2, 1, 3)
    assert checks_close(y, c.arrays["out"], RT, AT)


def test_attention_decode_is_last_causal_row(goldens):
    """One token against a cache == the last query row of causal attention (BTHD golden), and with grouped
    heads == attention on repeated key/value heads (F.repeatHeads)."""
    c = goldens["sdpa_bthd_causal"]
    for b in range(2):
        q = c.arrays["in0"][b, -1]           # [H, E]
        kc, vc = c.arrays["in1"][b], c.arrays["in2"][b]  # [S, H, E]
        y = oracle.attention_decode(q, kc, vc)
        assert checks_close(y, c.arrays["out"][b, -1], RT, AT)
    rng = np.random.default_rng(0)
    h, kv, s, d = 8, 2, 37, 16
    q = rng.standard_normal((h, d)).astype(np.float32)
    kc = rng.standard_normal((s, kv, d)).astype(np.float32)
    vc = rng.standard_normal((s, kv, d)).astype(np.float32)
    y = oracle.attention_decode(q, kc, vc)
    krep = np.repeat(kc, h // kv, axis=1).transpose(1, 0, 2)  # [H, S, D]
    vrep = np.repeat(vc, h // kv, axis=1).transpose(1, 0, 2)
    y2 = oracle.sdpa(q[:, None, :], krep, vrep, False)[:, 0, :]
    assert np.array_equal(y, y2)


def test_prefill_ref_is_decode_ref_token_by_token():
    """The many-token restatement used by the full-size prefill test is the decode oracle applied token by token: same
    cache rows, same last-token logits, up to the summation order of the FP64 accumulator of the linears."""
    import torch

    import quantizers
    from decode_oracle import SLOTS, decode_ref, prefill_ref
    from helpers import GGML_ID
    cfg = dict(layers=2, d_model=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=96, max_ctx=16, rms_eps=1e-5, rope_theta=5e5)
    g = torch.Generator().manual_seed(3)
    rng = np.random.default_rng(3)
    d, qd, kd, ffn = 256, 256, 128, 512
    shapes = {"attn_q": (qd, d), "attn_k": (kd, d), "attn_v": (kd, d), "attn_o": (d, qd), "ffn_gate": (ffn, d), "ffn_up": (ffn, d),
              "ffn_down": (d, ffn)}
    fmts = {"attn_q": "Q4_K", "attn_k": "Q4_K", "attn_v": "Q6_K", "attn_o": "Q4_0", "ffn_gate": "Q5_K", "ffn_up": "Q5_K", "ffn_down": "Q6_K"}
    layers = []
    for _ in range(2):
        L = {}
        for slot in SLOTS:
            n, k = shapes[slot]
            L[slot] = (GGML_ID[fmts[slot]], quantizers.quantize(fmts[slot], torch.randn(n, k, generator=g) * 0.05).numpy(), n, k)
        L["attn_norm"] = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        L["ffn_norm"] = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        layers.append(L)
    out_norm = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    out_w = (8, quantizers.quantize("Q8_0", torch.randn(96, d, generator=g) * 0.05).numpy(), 96, d)
    pos0, T = 3, 9
    k0 = np.zeros((2, 16, 2, 64), dtype=np.float32)
    v0 = np.zeros_like(k0)
    k0[:, :pos0] = rng.standard_normal(k0[:, :pos0].shape)
    v0[:, :pos0] = rng.standard_normal(v0[:, :pos0].shape)
    x = rng.standard_normal((T, d)).astype(np.float32)
    ka, va, kb, vb = k0.copy(), v0.copy(), k0.copy(), v0.copy()
    for t in range(T):
        ref = decode_ref(cfg, layers, out_norm, out_w, ka, va, x[t], pos0 + t)
    got = prefill_ref(cfg, layers, out_norm, out_w, kb, vb, x, pos0)
    assert np.abs(got - ref).max() <= 1e-6 * np.abs(ref).max()
    assert np.abs(ka - kb).max() <= 1e-6 * np.abs(ka).max() and np.abs(va - vb).max() <= 1e-6 * np.abs(va).max()
