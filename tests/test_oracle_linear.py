"""Pins the oracle's linear functions against the reference's goldens and its GgufChecks recipe."""
import numpy as np
import pytest

import ggml_numpy
from helpers import (GGML_ID, GGML_NAMES, GOLDEN_CODE_TO_GGML, HOT_FORMATS, JavaRandom, checks_close, java_string_hash, norm_err,
                     random_valid_blocks)
from oracle import oracle


def ulp_diff(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


def near(y, ref, bias):
    """Equal up to one FP32 rounding of the dot and one of the sum (a cancelling bias makes that many ulps)."""
    slack = 2.0 ** -23 * (np.abs(ref.astype(np.float64)) + 2 * np.abs(bias.astype(np.float64))[None, :])
    return bool(np.all(np.abs(y.astype(np.float64) - ref) <= slack))


@pytest.mark.parametrize("code", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("rows", [1, 5, 40])
def test_golden_linear(goldens, code, rows):
    """gguf_linear_* (Golden.java:321-322): out = x W^T + b from torch in FP64.  The reference's bar is
    rtol 1e-4 / atol 1e-3 (Golden.java:483-498); the oracle rounds the dot to FP32 before the FP32 bias
    add (Gguf.java:97) where the golden rounds once: the two differ by at most one rounding of the dot
    (2^-24 |dot|) plus one of the sum."""
    fid = GOLDEN_CODE_TO_GGML[code]
    case = goldens[f"gguf_linear_{GGML_NAMES[fid].lower()}_r{rows}"]
    x, raw, bias, out = case.arrays["in0"], case.arrays["in1"].astype(np.uint8), case.arrays["in2"], case.arrays["out"]
    n = int(case.attrs[1])
    assert out.shape == (rows, n)
    y = oracle.gguf_linear(fid, x, raw, bias, n, 512)
    assert checks_close(y, out, 1e-4, 1e-3)
    assert near(y, out, bias)
    # without the second rounding the golden is reproduced exactly: (float)(fp64 dot + bias)
    w = oracle.dequantize(fid, raw, n * 512).reshape(n, 512).astype(np.float64)
    exact = (x.astype(np.float64) @ w.T + bias.astype(np.float64)).astype(np.float32)
    assert ulp_diff(exact, out).max() <= 1  # numpy's fp64 summation order differs from torch's in the last bit at most


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_ggufchecks_recipe(gguf_fixture, fmt):
    """GgufChecks.check (GgufChecks.java:82-103): x from java.util.Random(type.hashCode()) for 1, 5, 40 rows drawn
    from one generator, bias {0.25,-0.5,1}, reference = FP64 dot over expect.<T>; bar 2e-4 * max."""
    raw = gguf_fixture.raw(f"w.{fmt}")
    expect = gguf_fixture.f32(f"expect.{fmt}").astype(np.float64)
    rnd = JavaRandom(java_string_hash(fmt))
    bias = np.array([0.25, -0.5, 1.0], dtype=np.float32)
    for rows in (1, 5, 40):
        x = np.array([rnd.next_float() * np.float32(2) - np.float32(1) for _ in range(rows * 512)], dtype=np.float32).reshape(rows, 512)
        ref = (bias.astype(np.float64)[None, :] + x.astype(np.float64) @ expect.T).astype(np.float32)
        y = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, 3, 512)
        assert norm_err(y, ref) <= 2e-4
        assert near(y, ref, bias)


def test_java_random_known_values():
    """JDK-documented first outputs of new Random(42): nextInt() = -1170105035, 234785527."""
    r = JavaRandom(42)
    v = r.next(32)
    assert (v - (1 << 32) if v >= (1 << 31) else v) == -1170105035
    assert r.next(32) == 234785527
    assert java_string_hash("hello") == 99162322 and java_string_hash("Q4_K") == 81 * 31 ** 3 + 52 * 31 ** 2 + 95 * 31 + 75


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_unit_vectors_give_columns(fmt):
    """x = e_j turns the GEMV into column j of the dequantised matrix, bit for bit (addressing check)."""
    rng = np.random.default_rng(11)
    n, k = 5, 512
    raw = random_valid_blocks(rng, fmt, n, k)
    w = ggml_numpy.dequant(fmt, raw).reshape(n, k)
    cols = [0, 1, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, 300, 511]
    x = np.zeros((len(cols), k), dtype=np.float32)
    for r, j in enumerate(cols):
        x[r, j] = 1.0
    y = oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)
    assert np.array_equal(y.view(np.uint32), w[:, cols].T.copy().view(np.uint32))


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_linear_against_fp64_numpy(fmt):
    rng = np.random.default_rng(5)
    n, k, rows = 17, 1024, 3
    raw = random_valid_blocks(rng, fmt, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    w = ggml_numpy.dequant(fmt, raw).reshape(n, k).astype(np.float64)
    dot = x.astype(np.float64) @ w.T
    y = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k)
    if fmt == "Q8_0":
        ref = (dot + bias).astype(np.float32)
    else:
        ref = dot.astype(np.float32) + bias
    assert near(y, ref, bias)
    # all-ones input -> row sums (+bias)
    ones = np.ones((1, k), dtype=np.float32)
    y1 = oracle.gguf_linear(GGML_ID[fmt], ones, raw, None, n, k)
    assert ulp_diff(y1[0], w.sum(axis=1).astype(np.float32)).max() <= 1


def test_matmul_goldens(goldens):
    for name in ("matmul_t01_17x33x9", "matmul_t01_1x1x1", "matmul_t01_40x3x70"):
        c = goldens[name]
        y = oracle.matmul_nt(c.arrays["in0"], c.arrays["in1"])
        assert checks_close(y, c.arrays["out"], 1e-4, 1e-4)
        assert ulp_diff(y, c.arrays["out"]).max() <= 1


def test_quantize_q8_0_invariants():
    """Quant.Quantize.reference semantics (Quant.java:102-118); exact bytes on .5 ties are parity-unpinned
    (no reference-held vector of quantiser output), so this checks the closed form and its invariants,
    including the reference's own round-trip bar (OpsAccelTest.java:261-267: one step 1/127 + 1e-6)."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal(32 * 200).astype(np.float32)
    x[:32] = 0  # zero block
    x[32:64] = np.linspace(-1, 1, 32)  # max maps to +-127
    q = oracle.quantize_q8_0(x)
    b = q.reshape(-1, 34)
    d16 = b[:, :2].copy().view(np.float16)[:, 0]
    qs = b[:, 2:].view(np.int8)
    assert d16[0] == 0 and not qs[0].any()
    assert qs[1].min() == -127 and qs[1].max() == 127
    amax = np.abs(x.reshape(-1, 32)).max(axis=1).astype(np.float64)
    d32 = (amax / 127.0).astype(np.float32)
    assert np.array_equal(d16, d32.astype(np.float16))
    # closed form, computed independently in numpy with round-half-away
    s = np.divide(x.reshape(-1, 32).astype(np.float64), d32.astype(np.float64)[:, None], out=np.zeros((200, 32)), where=d32[:, None] > 0)
    exp = np.clip(np.sign(s) * np.floor(np.abs(s) + 0.5), -127, 127).astype(np.int8)
    assert np.array_equal(qs, exp)
    dq = oracle.dequantize(8, q, x.size).reshape(-1, 32)
    step = amax / 127.0
    assert np.all(np.abs(dq - x.reshape(-1, 32)) <= (step * (0.5 + 127 * 2.0 ** -11) + 1e-12)[:, None])
    scale = np.abs(x).max()
    assert np.abs(dq.reshape(-1) - x).max() <= scale * (1 / 127.0) + 1e-6


def test_quantize_q8_0_ties_round_half_away_from_zero_literals():
    """Quant.java:113-114 rounds s = x / d half away from zero (Math.round on the magnitude, sign restored) and clamps to +-127.
    A block whose largest magnitude is 127 has d = (float)(127 / 127.0) = 1, so the quotients are the inputs themselves: the
    expected bytes below are written out as numbers, not recomputed.  Round-half-even would give 0, 2, 2 for 0.5, 1.5, 2.5
    and 126 for 126.5."""
    x = np.zeros(64, dtype=np.float32)
    x[:9] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    x[32:41] = [-127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]   # the same with the maximum on the negative side
    q = oracle.quantize_q8_0(x).reshape(2, 34)
    for b in range(2):
        assert q[b, :2].copy().view(np.float16)[0] == np.float16(1.0)
        qs = q[b, 2:].view(np.int8)
        assert qs[0] == (127 if b == 0 else -127)
        assert list(qs[1:9]) == [1, 2, 3, -1, -2, -3, 127, -127]
        assert not qs[9:].any()
    # one float below / above a tie falls to the nearer integer
    y = np.zeros(32, dtype=np.float32)
    y[:5] = [127.0, np.nextafter(np.float32(2.5), np.float32(0)), np.nextafter(np.float32(2.5), np.float32(3)),
             np.nextafter(np.float32(-0.5), np.float32(0)), np.nextafter(np.float32(-0.5), np.float32(-1))]
    assert list(oracle.quantize_q8_0(y).reshape(34)[2:].view(np.int8)[:5]) == [127, 2, 3, 0, -1]


def test_cpu_dequant_gemm_baseline_agrees_with_the_oracle():
    """The C restatement of the reference's dequantise + GEMM branch (the CPU baseline of the many-row configurations)
    against the FP64 oracle on the same blocks: equal within FP32 rounding of a K-blocked FMA sum, at ragged sizes (edge
    panels in both directions, K past one block of 256), for one thread and for several."""
    from oracle import oracle
    rng = np.random.default_rng(77)
    for fmt, n, k, rows in (("Q4_K", 70, 768, 13), ("Q6_K", 33, 512, 40), ("Q4_0", 129, 96, 7), ("Q8_0", 16, 32, 1)):
        raw = random_valid_blocks(rng, fmt, n, k)
        x = rng.standard_normal((rows, k)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k)
        for threads in (1, 3):
            y, t_deq, t_mm = oracle.dequant_gemm(GGML_ID[fmt], x, raw, bias, n, k, threads)
            assert norm_err(y, ref) <= 2e-6, (fmt, threads, norm_err(y, ref))
            assert t_deq >= 0 and t_mm >= 0
    assert oracle.cpu_vector_lanes() in (4, 8, 16) and oracle.cpu_threads() >= 1
