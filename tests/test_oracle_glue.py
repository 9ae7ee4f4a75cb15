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
