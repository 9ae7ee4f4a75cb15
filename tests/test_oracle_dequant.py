"""Pins the oracle's dequantisers (oracle/jitnn_oracle.c) bit-exactly against the reference's own fixtures."""
import numpy as np
import pytest

import ggml_numpy
from helpers import BLOCK, GGML_ID, GOLDEN_CODE_TO_GGML, GGML_NAMES, random_valid_blocks
from oracle import oracle

ALL = ["Q8_0", "Q4_0", "Q4_1", "Q4_K", "Q5_K", "Q6_K", "Q5_0", "Q5_1", "Q2_K", "Q3_K"]


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("fmt", ALL)
def test_fixture_gguf_expect_bit_exact(gguf_fixture, fmt):
    """w.<T> dequantises to expect.<T> (llama.cpp's gguf package output) - GgufChecks.java:75-80, here bit for bit."""
    raw = gguf_fixture.raw(f"w.{fmt}")
    expect = gguf_fixture.f32(f"expect.{fmt}")
    assert expect.shape == (3, 512)
    got = oracle.dequantize(GGML_ID[fmt], raw, 3 * 512)
    assert np.array_equal(bits(got), bits(expect.reshape(-1)))


@pytest.mark.parametrize("code", [0, 1, 2, 3, 4])
def test_golden_dequant_bit_exact(goldens, code):
    fmt = GGML_NAMES[GOLDEN_CODE_TO_GGML[code]]
    case = goldens[f"gguf_dequant_{fmt.lower()}"]
    raw = case.arrays["in0"].astype(np.uint8)
    out = case.arrays["out"]
    got = oracle.dequantize(GOLDEN_CODE_TO_GGML[code], raw, out.size)
    assert np.array_equal(bits(got), bits(out.reshape(-1)))


@pytest.mark.parametrize("fmt", ALL)
def test_oracle_vs_independent_numpy_on_random_bytes(fmt):
    """Every byte value in every position (fully random bytes incl. scales that decode to inf/nan/subnormals
    are excluded by keeping FP16 scale fields finite): division/remainder form == shift/mask form."""
    rng = np.random.default_rng(1234 + GGML_ID[fmt])
    raw = random_valid_blocks(rng, fmt, 64, 1024, lo=1e-6, hi=4.0)
    got = oracle.dequantize(GGML_ID[fmt], raw, 64 * 1024)
    exp = ggml_numpy.dequant(fmt, raw)
    assert np.array_equal(bits(got), bits(exp))


@pytest.mark.parametrize("fmt", ALL)
def test_each_byte_position_takes_all_values(fmt):
    """One block, one byte swept over 0..255 at every payload position: catches a wrong index or nibble."""
    qk, nb = BLOCK[fmt]
    rng = np.random.default_rng(7)
    base = random_valid_blocks(rng, fmt, 1, qk)
    scale_bytes = {"Q8_0": {0, 1}, "Q4_0": {0, 1}, "Q4_1": {0, 1, 2, 3}, "Q5_0": {0, 1}, "Q5_1": {0, 1, 2, 3}, "Q4_K": {0, 1, 2, 3},
                   "Q5_K": {0, 1, 2, 3}, "Q6_K": {208, 209}, "Q2_K": {80, 81, 82, 83}, "Q3_K": {108, 109}}[fmt]
    blocks = []
    for pos in range(nb):
        if pos in scale_bytes:
            continue
        for v in range(0, 256, 5):
            b = base.copy()
            b[pos] = v
            blocks.append(b)
    raw = np.concatenate(blocks)
    n = len(blocks) * qk
    assert np.array_equal(bits(oracle.dequantize(GGML_ID[fmt], raw, n)), bits(ggml_numpy.dequant(fmt, raw)))


def test_half_conversions_match_numpy():
    h = np.arange(65536, dtype=np.uint16)
    ref = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.half_to_float(int(v)) for v in h], dtype=np.float32)
    finite = ~np.isnan(ref)
    assert np.array_equal(bits(got[finite]), bits(ref[finite]))
    assert np.all(np.isnan(got[~finite]))
    # encode: every half round-trips; random floats agree with numpy's round-to-nearest-even
    back = np.array([oracle.float_to_half(float(v)) for v in ref[finite]], dtype=np.uint16)
    assert np.array_equal(back, h[finite])
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
                         np.array([65504, 65519.99, 65520, 1e9, 6.1e-5, 5.96e-8, 2.98e-8, 2.9802322e-08, 3e-8, 0.0, -0.0], dtype=np.float32)])
    # midpoints between neighbouring halves (ties)
    mids = ((ref[finite][:-1].astype(np.float64) + ref[finite][1:].astype(np.float64)) / 2).astype(np.float32)
    xs = np.concatenate([xs, mids[np.isfinite(mids)][::7]])
    with np.errstate(over="ignore"):
        exp = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float_to_half(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(got, exp)


def test_block_metadata():
    for fmt, (qk, nb) in BLOCK.items():
        assert oracle.block_values(GGML_ID[fmt]) == qk
        assert oracle.block_bytes(GGML_ID[fmt]) == nb
    assert oracle.block_values(99) == 0
