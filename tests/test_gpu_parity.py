"""Parity of the HIP path (through the C ABI) with the CPU oracle, the reference's golden vectors and its
GgufChecks recipe.  Bars: dequantised weights bit-exact; GEMV max|y-ref| / max|ref| <= 1e-4 (the
normalisation of GgufChecks.close, GgufChecks.java:110-120) and the goldens' own rtol 1e-4 / atol 1e-3
(Golden.java:483-498)."""
import numpy as np
import pytest

import ggml_numpy
from helpers import (BLOCK, GGML_ID, GGML_NAMES, GOLDEN_CODE_TO_GGML, HOT_FORMATS, JavaRandom, checks_close, java_string_hash, norm_err,
                     random_valid_blocks)

pytestmark = pytest.mark.gpu

GEMV_BAR = 1e-4    # up to 64 rows: FP32 GEMV kernels (this covers every row count the reference's own tests use)
MFMA_BAR = 2e-3    # more rows (prefill): FP16 MFMA kernel


def bar(rows):
    return GEMV_BAR if rows <= 64 else MFMA_BAR


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def weight(jn, fmt, raw, n, k):
    return jn.Tensor.quantized(jn.DType[fmt], raw, n, k)


# ------------------------------------------------------------------------------------------ dequantise

@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_dequant_fixture_bit_exact(jn, gguf_fixture, fmt):
    """GgufChecks.check 'values' and 'dequantize' (GgufChecks.java:75-80) - here bit for bit."""
    w = weight(jn, fmt, gguf_fixture.raw(f"w.{fmt}"), 3, 512)
    expect = gguf_fixture.f32(f"expect.{fmt}").reshape(-1)
    assert np.array_equal(bits(w.to_float_array()), bits(expect))
    d = jn.Quant.dequantize(w) if fmt == "Q8_0" else jn.Gguf.dequantize(w)
    assert np.array_equal(bits(d.numpy().reshape(-1)), bits(expect))


@pytest.mark.parametrize("code", [0, 1, 2, 3, 4])
def test_dequant_goldens_bit_exact(jn, goldens, code):
    fmt = GGML_NAMES[GOLDEN_CODE_TO_GGML[code]]
    case = goldens[f"gguf_dequant_{fmt.lower()}"]
    w = weight(jn, fmt, case.arrays["in0"].astype(np.uint8), 3, 512)
    assert np.array_equal(bits(w.to_float_array()), bits(case.arrays["out"].reshape(-1)))


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_dequant_random_blocks_vs_oracle(jn, fmt):
    from oracle import oracle
    rng = np.random.default_rng(100 + GGML_ID[fmt])
    n, k = 33, 1024
    raw = random_valid_blocks(rng, fmt, n, k, lo=1e-6, hi=4.0)  # includes FP16-subnormal scales
    got = weight(jn, fmt, raw, n, k).to_float_array()
    assert np.array_equal(bits(got), bits(oracle.dequantize(GGML_ID[fmt], raw, n * k)))


# ------------------------------------------------------------------------------------------ linear, reference fixtures

@pytest.mark.parametrize("code", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("rows", [1, 5, 40])
def test_linear_goldens(jn, goldens, code, rows):
    fid = GOLDEN_CODE_TO_GGML[code]
    fmt = GGML_NAMES[fid]
    case = goldens[f"gguf_linear_{fmt.lower()}_r{rows}"]
    x, raw, bias, out = case.arrays["in0"], case.arrays["in1"].astype(np.uint8), case.arrays["in2"], case.arrays["out"]
    n = int(case.attrs[1])
    y = jn.Gguf.linear(jn.Tensor.of(x), weight(jn, fmt, raw, n, 512), jn.Tensor.of(bias)).numpy()
    assert y.shape == out.shape
    assert checks_close(y, out, 1e-4, 1e-3)
    assert norm_err(y, out) <= bar(rows)


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_linear_ggufchecks_recipe(jn, gguf_fixture, fmt):
    """GgufChecks.check (GgufChecks.java:82-103): 1, 5 and 40 rows from one java.util.Random, bias, 2e-4 * max."""
    from oracle import oracle
    raw = gguf_fixture.raw(f"w.{fmt}")
    expect = gguf_fixture.f32(f"expect.{fmt}").astype(np.float64)
    w = weight(jn, fmt, raw, 3, 512)
    rnd = JavaRandom(java_string_hash(fmt))
    bias = np.array([0.25, -0.5, 1.0], dtype=np.float32)
    for rows in (1, 5, 40):
        x = np.array([rnd.next_float() * np.float32(2) - np.float32(1) for _ in range(rows * 512)], dtype=np.float32).reshape(rows, 512)
        ref = (bias.astype(np.float64)[None, :] + x.astype(np.float64) @ expect.T).astype(np.float32)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias)).numpy()
        assert norm_err(y, ref) <= 2e-4, (fmt, rows, norm_err(y, ref))
        assert norm_err(y, oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, 3, 512)) <= bar(rows)


# ------------------------------------------------------------------------------------------ linear, seeded inputs vs oracle

SHAPES = [  # (n, k): ragged row counts, one block, several wave steps, K past one LDS chunk
    (1, 256), (7, 512), (37, 1024), (64, 4096), (131, 4096), (29, 14336), (5, 8192 + 256),
]


@pytest.mark.parametrize("fmt", HOT_FORMATS)
@pytest.mark.parametrize("n,k", SHAPES)
def test_gemv_vs_oracle(jn, fmt, n, k):
    from oracle import oracle
    rng = np.random.default_rng(n * 100003 + k + GGML_ID[fmt])
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    for rows in (1, 2, 3, 4, 8):
        x = rng.standard_normal((rows, k)).astype(np.float32)
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias if rows % 2 else None, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias) if rows % 2 else None).numpy()
        assert y.shape == (rows, n)
        assert norm_err(y, ref) <= GEMV_BAR, (fmt, n, k, rows, norm_err(y, ref))


@pytest.mark.parametrize("k", [256, 1024, 4096])
def test_q6k_many_rows_integer_variant(jn, k):
    """A tall Q6_K matrix (many turns per workgroup, a row count that is no multiple of four) through the INT8
    matrix-core kernel - activations as 22-bit fixed point in three byte planes - with rows of 256 (one wave, more
    outputs per flush than threads), 1024 and longer: same bar, and in fact FP32-grade error, on ordinary,
    outlier-ridden, tiny, partly zero and unit-vector activations, with and without bias."""
    from oracle import oracle
    rng = np.random.default_rng(4242 + k)
    n = 16 * 2048 + 37
    raw = random_valid_blocks(rng, "Q6_K", n, k)
    w = weight(jn, "Q6_K", raw, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    xs = []
    xs.append(rng.standard_normal(k).astype(np.float32))
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, size=max(1, k // 128))] *= np.float32(1e4)   # outliers share their 64-value unit with ordinary values
    xs.append(x)
    xs.append((rng.standard_normal(k) * 1e-30).astype(np.float32))    # near the bottom of the FP32 range
    x = rng.standard_normal(k).astype(np.float32)
    x[: k // 2] = 0.0                                                  # whole units of zeros
    x[k // 2: k // 2 + 64] *= np.float32(1e-20)
    xs.append(x)
    x = np.zeros(k, dtype=np.float32)
    x[k - 3] = 1.0                                                     # a column of the dequantised matrix
    xs.append(x)
    for i, x in enumerate(xs):
        b = bias if i % 2 else None
        ref = oracle.gguf_linear(14, x[None, :], raw, b, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x[None, :]), w, jn.Tensor.of(b) if b is not None else None).numpy()
        assert y.shape == (1, n)
        err = norm_err(y, ref) if b is None else norm_err(y - b, ref - b)
        assert err <= GEMV_BAR, (k, i, err)
        assert err <= 5e-6, (k, i, err)   # what the variant actually delivers
    col = jn.Gguf.linear(jn.Tensor.of(xs[4][None, :]), w, None).numpy()[0]
    deq = w.to_float_array().reshape(n, k)[:, k - 3]
    assert np.allclose(col, deq, rtol=3e-7, atol=0.0)


@pytest.mark.parametrize("fmt", HOT_FORMATS)
@pytest.mark.parametrize("rows", [2, 5, 7, 8])
def test_batch_rows_of_very_different_magnitude(jn, fmt, rows):
    """Batches 2..8 with K a multiple of 256 run on the matrix cores with the activations split into two FP16 parts
    under a power-of-two scale per (row, 256-value column): huge, tiny, zero and outlier-dominated rows must each
    meet the GEMV bar against their own largest output."""
    from oracle import oracle
    rng = np.random.default_rng(rows * 31 + GGML_ID[fmt])
    n, k = 83, 2048 + 256
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0] *= np.float32(1e6)
    x[1] *= np.float32(1e-6)
    if rows > 2:
        x[2] = 0
    if rows > 3:
        x[3, 700] = np.float32(1e4)     # one outlier in a column of ordinary values
    if rows > 4:
        x[4, :256] *= np.float32(1e-30)  # a column near the bottom of the FP32 range
    ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)
    y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
    for r in range(rows):
        scale = max(float(np.abs(ref[r]).max()), 1e-30)
        assert float(np.abs(y[r].astype(np.float64) - ref[r]).max()) / scale <= GEMV_BAR, (fmt, rows, r)
    if rows > 2:
        assert not y[2].any()


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_small_k_32_blocks_and_many_rows(jn, fmt):
    """K of a single block for the 32-value formats; rows beyond one batch of 8 (9, 17, 40, 64)."""
    from oracle import oracle
    rng = np.random.default_rng(77)
    k = 32 * 3 if fmt in ("Q8_0", "Q4_0", "Q4_1") else 256
    n = 19
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    for rows in (9, 17, 40, 64):
        x = rng.standard_normal((rows, k)).astype(np.float32)
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
        assert norm_err(y, ref) <= bar(rows), (fmt, rows, norm_err(y, ref))


@pytest.mark.parametrize("fmt", ["Q4_K", "Q5_K", "Q6_K", "Q4_0", "Q4_1", "Q8_0", "Q5_1", "Q2_K"])
@pytest.mark.parametrize("n,k", [(16, 256), (100, 2048), (1000, 4096 + 256), (259, 14336)])
def test_one_pass_rows_kernel(jn, fmt, n, k):
    """9..64 rows take one pass over the weights (K-quants: block scales folded into FP16 weight operands; 32-value
    formats: the quants as operands, every block's sum scaled on its own; the activations split hi + lo): whole and
    ragged tiles of 16 weight rows, one to many 256-value columns, every number of groups of eight rows, bias, and
    activation rows of very different magnitudes - bar 1e-4 of the largest output per row.  (Q5_1 - a Q4_1 tile with a
    fifth bit - and Q2_K - Q6_K's element order, 4-bit scales and minima - take this kernel from five rows.)"""
    from oracle import oracle
    rng = np.random.default_rng(n + k + GGML_ID[fmt])
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    for rows in ((5, 8) if fmt in ("Q5_1", "Q2_K") else ()) + (9, 16, 24, 33, 40, 57, 64):
        x = rng.standard_normal((rows, k)).astype(np.float32)
        x[1] *= np.float32(1e6)
        x[2] *= np.float32(1e-6)
        x[3] = 0
        x[4, rng.integers(0, k, size=max(1, k // 256))] *= np.float32(1e4)
        x[rows - 1] *= np.float32(1e-30)
        b = bias if rows % 2 == 0 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, b, n, k).astype(np.float64)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(b) if b is not None else None).numpy()
        for r in range(rows):
            scale = max(float(np.abs(ref[r]).max()), 1e-37)
            assert float(np.abs(y[r].astype(np.float64) - ref[r]).max()) / scale <= GEMV_BAR, (fmt, n, k, rows, r)
        assert not y[3].any() if b is None else np.array_equal(y[3], bias)


@pytest.mark.parametrize("fmt", ["Q4_0", "Q4_1", "Q8_0"])
@pytest.mark.parametrize("k", [96, 160])
def test_odd_block_counts_at_every_batch_size(jn, fmt, k):
    """Rows of 3 and 5 blocks (no pairs of blocks, no whole 256-value columns) at 1..8 rows: the single-block variants of
    the register kernels and of the kernel with the activations in LDS."""
    from oracle import oracle
    rng = np.random.default_rng(k + GGML_ID[fmt])
    n = 45
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    for rows in range(1, 9):
        x = rng.standard_normal((rows, k)).astype(np.float32)
        b = bias if rows % 2 == 0 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, b, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(b) if b is not None else None).numpy()
        assert norm_err(y, ref) <= GEMV_BAR, (fmt, k, rows, norm_err(y, ref))


PREFILL_SHAPES = [  # (n, k, rows): ragged tiles in every dimension, K past one step, K split into 8 and into 4 slices,
    # and (130 x 4352) into four slices of unequal length: 17 blocks of 256 over slices of whole blocks
    (256, 1024, 65), (131, 4096, 200), (64, 14336, 97), (130, 512, 129), (1, 256, 70), (384, 4096, 513), (130, 4352, 129),
    (40, 16640, 70),  # rows longer than the one-launch activation preparation takes: scale and conversion in two launches
]


@pytest.mark.parametrize("fmt", HOT_FORMATS)
@pytest.mark.parametrize("n,k,rows", PREFILL_SHAPES)
def test_prefill_mfma_vs_oracle(jn, fmt, n, k, rows):
    """More than 64 rows run the dequantise-to-LDS MFMA kernel (FP16 operands, FP32 accumulation): bar 2e-3."""
    from oracle import oracle
    rng = np.random.default_rng(n * 7 + k + rows + GGML_ID[fmt])
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0] *= 1e4      # rows of very different magnitude: the per-row FP16 scale must cope
    x[1] *= 1e-6
    bias = rng.standard_normal(n).astype(np.float32)
    ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k)
    y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias)).numpy()
    assert y.shape == (rows, n)
    # row by row (a tiny row must not hide behind a huge one), against the larger of the row's biggest output and the
    # typical output magnitude |x_r| * rms row norm of W (one output alone can be small by cancellation)
    wnorm = float(np.sqrt((ggml_numpy.dequant(fmt, raw).astype(np.float64) ** 2).sum() / n))
    for r in range(rows):
        scale = max(float(np.abs(ref[r] - bias).max()), float(np.linalg.norm(x[r].astype(np.float64))) * wnorm, 1e-30)
        assert np.abs(y[r] - ref[r]).max() <= MFMA_BAR * scale + 1e-6 * np.abs(bias).max(), (fmt, r)


@pytest.mark.parametrize("fmt", ["Q4_0", "Q8_0", "Q4_1"])
@pytest.mark.parametrize("n,k,rows", [(40, 32 * 7, 70), (132, 4096 + 32, 300)])  # the second: few tiles, so K is split into slices
def test_prefill_k_tail_of_32(jn, fmt, n, k, rows):
    from oracle import oracle
    rng = np.random.default_rng(3)
    raw = random_valid_blocks(rng, fmt, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    y = jn.Gguf.linear(jn.Tensor.of(x), weight(jn, fmt, raw, n, k), None).numpy()
    assert norm_err(y, oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)) <= MFMA_BAR


@pytest.mark.parametrize("fmt", HOT_FORMATS)
def test_unit_vectors_give_columns(jn, fmt):
    """x = e_j reduces the GEMV to column j of the dequantised matrix: catches any misplaced value."""
    rng = np.random.default_rng(11)
    n, k = 9, 1024
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    wd = ggml_numpy.dequant(fmt, raw).reshape(n, k)
    cols = np.concatenate([np.arange(0, 64), np.arange(250, 262), np.arange(500, 520), np.array([767, 768, 1023])])
    for c0 in range(0, len(cols), 8):
        cc = cols[c0:c0 + 8]
        x = np.zeros((len(cc), k), dtype=np.float32)
        x[np.arange(len(cc)), cc] = 1.0
        y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
        exp = wd[:, cc].T
        assert np.allclose(y, exp, rtol=3e-7, atol=1e-9), (fmt, cc)


def test_batched_leading_axes(jn):
    """x [2, 3, K] -> y [2, 3, N] (Gguf.linear keeps the leading axes, Gguf.java:86-93)."""
    from oracle import oracle
    rng = np.random.default_rng(5)
    n, k = 24, 512
    raw = random_valid_blocks(rng, "Q5_K", n, k)
    x = rng.standard_normal((2, 3, k)).astype(np.float32)
    y = jn.Gguf.linear(jn.Tensor.of(x), weight(jn, "Q5_K", raw, n, k), None).numpy()
    assert y.shape == (2, 3, n)
    assert norm_err(y.reshape(6, n), oracle.gguf_linear(13, x.reshape(6, k), raw, None, n, k)) <= GEMV_BAR


# ------------------------------------------------------------------------------------------ Q8_0 quantiser

def test_quantize_q8_0_bit_exact_vs_oracle(jn):
    """Same bytes as the oracle's restatement of Quant.Quantize.reference (exact bytes on .5 ties are not pinned by
    any reference-held vector; both sides share the closed form)."""
    from oracle import oracle
    rng = np.random.default_rng(21)
    x = (rng.standard_normal((64, 256)) * rng.uniform(1e-3, 50, size=(64, 1))).astype(np.float32)
    x[0, :32] = 0
    x[1, :32] = np.linspace(-3, 3, 32)
    x[2, :32] = 1e-7   # scale below the FP16 normal range
    x[3, :32] = np.arange(32) * 0.5  # exact .5 ties after scaling by a power-of-two-friendly d
    q = jn.Quant.quantize_q8(jn.Tensor.of(x))
    assert q.shape() == (64, 256) and q.dtype() == jn.DType.Q8_0
    exp = oracle.quantize_q8_0(x)
    got = q.to_float_array()
    assert np.array_equal(bits(got), bits(oracle.dequantize(8, exp, x.size)))
    # round trip within one step, the reference's own bar (OpsAccelTest.java:261-267)
    assert np.abs(got - x.reshape(-1)).max() <= np.abs(x).max() * (1 / 127.0) + 1e-6
    # and the linear on it agrees with the reference's FP64 host loop
    xin = rng.standard_normal((3, 256)).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    y = jn.F.linear_q8(jn.Tensor.of(xin), q, jn.Tensor.of(b)).numpy()
    assert norm_err(y, oracle.gguf_linear(8, xin, exp, b, 64, 256)) <= 1e-5


def test_quantize_q8_0_bytes_on_ties_extremes_and_ragged_sizes(jn):
    """The quantiser's bytes against the oracle's on what its short form must get right: values on and one float either
    side of every half-integer multiple of the block's scale, blocks whose scale is huge, tiny, subnormal or zero, and
    sizes that are not whole groups of 64 blocks.  (Values that are not finite are outside the reference's tests, and the C
    oracle's cast of NaN to an integer is not Java's.)"""
    import ctypes as C
    from jitnn_amd import _lib
    from oracle import oracle
    rng = np.random.default_rng(33)
    rows = []
    for amax in (127.0, 1.0, 3.1415927, 1e-3, 6.5e4, 1e20, 1e-20, 2.0 ** -99, 2.0 ** -101, 1e-38, 1e-42, 3e38):
        d = np.float32(np.float64(np.float32(amax)) / 127.0)
        for _ in range(3):
            ks = rng.integers(0, 127, size=31)
            ties = ((ks + 0.5) * np.float64(d)).astype(np.float32)
            ties = np.nextafter(ties, np.float32(rng.choice([-np.inf, np.inf])) if rng.integers(3) else ties).astype(np.float32)
            blk = np.concatenate([[np.float32(amax)], ties * rng.choice([-1, 1], size=31).astype(np.float32)])
            rows.append(rng.permutation(blk).astype(np.float32))
    rows.append(np.zeros(32, dtype=np.float32))
    rows.append(np.full(32, -0.0, dtype=np.float32))
    special = np.stack(rows)
    bulk = (rng.standard_normal((64 * 5 + 37, 32)) * 10.0 ** rng.uniform(-6, 6, size=(64 * 5 + 37, 1))).astype(np.float32)
    x = np.concatenate([special, bulk])
    for count in (x.shape[0], 64, 65, 1, 200):
        xs = np.ascontiguousarray(x[:count])
        got = np.empty(xs.size // 32 * 34, dtype=np.uint8)
        rc = _lib.lib.jitnn_hip_quantize_q8_0(xs.ctypes.data_as(C.c_void_p), xs.size, got.ctypes.data_as(C.c_void_p))
        assert rc == 0 and np.array_equal(got, oracle.quantize_q8_0(xs)), count


# ------------------------------------------------------------------------------------------ the other dequantisable formats

# Q5_1, Q2_K: bit-exact dequantiser, plain GEMV up to 64 rows, a decoder of their own in the many-row kernel beyond.  Q5_0,
# Q3_K: rewritten at upload into Q8_0 / Q6_K blocks of exactly the same values, and from there on those formats' kernels.
EXTRA_FORMATS = ["Q5_0", "Q5_1", "Q2_K", "Q3_K"]
REWRITTEN = {"Q5_0": "Q8_0", "Q3_K": "Q6_K"}


@pytest.mark.parametrize("fmt", EXTRA_FORMATS)
def test_extra_format_dequant_fixture_bit_exact(jn, gguf_fixture, fmt):
    """w.<T> of the reference's fixture.gguf dequantises to expect.<T> bit for bit (GgufChecks.java:58-75)."""
    got = weight(jn, fmt, gguf_fixture.raw("w." + fmt), 3, 512).to_float_array()
    expect = gguf_fixture.f32("expect." + fmt).reshape(-1)
    assert np.array_equal(bits(got), bits(expect))


@pytest.mark.parametrize("fmt", EXTRA_FORMATS)
def test_extra_format_dequant_and_linear_vs_oracle(jn, fmt):
    from oracle import oracle
    rng = np.random.default_rng(500 + GGML_ID[fmt])
    n, k = 37, 1024
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    assert np.array_equal(bits(w.to_float_array()), bits(oracle.dequantize(GGML_ID[fmt], raw, n * k)))
    bias = rng.standard_normal(n).astype(np.float32)
    for rows in (1, 3, 8, 11, 40, 70, 300):  # 70, 300: past the GEMV range - the many-row kernel decodes Q5_1 and Q2_K itself
        x = rng.standard_normal((rows, k)).astype(np.float32)
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias if rows % 2 else None, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias) if rows % 2 else None).numpy()
        assert y.shape == (rows, n)
        bar = 2e-3 if rows > 64 else GEMV_BAR  # (the many-row kernel's FP16 operands)
        assert norm_err(y, ref) <= bar, (fmt, rows, norm_err(y, ref))


def test_batch_1_and_2_random_shapes_all_formats(jn):
    """Forty seeded shapes - any row count from 1 to 300, row lengths of 1 to 16 waves of the INT8 matrix-core kernel and lengths
    it does not take (odd multiples of 32 for the 32-value formats), one or two activation rows, with and without bias, all
    eight formats that kernel has units for - against the oracle."""
    from oracle import oracle
    rng = np.random.default_rng(20261)
    fmts = ["Q4_K", "Q5_K", "Q6_K", "Q4_0", "Q4_1", "Q8_0", "Q5_1", "Q2_K"]
    for case in range(40):
        fmt = fmts[case % len(fmts)]
        kq = 32 if fmt in ("Q4_0", "Q4_1", "Q8_0", "Q5_1") else 256
        k = kq * int(rng.integers(1, 16384 // kq + 1)) if case % 5 else kq * int(rng.integers(1, 9))
        n = int(rng.integers(1, 301))
        rows = 1 + case % 2
        raw = random_valid_blocks(rng, fmt, n, k)
        w = weight(jn, fmt, raw, n, k)
        x = rng.standard_normal((rows, k)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32) if case % 3 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias) if bias is not None else None).numpy()
        assert y.shape == (rows, n)
        assert norm_err(y, ref) <= GEMV_BAR, (case, fmt, n, k, rows, norm_err(y, ref))


def test_random_shapes_any_row_count_all_formats(jn):
    """Eighty seeded linears - one to 80 activation rows, one to 700 weight rows, rows of whole 256-value columns up to 16128
    values and of any whole number of blocks up to 8192, one activation row in four scaled by 1e5, with and without bias, all
    ten block formats - against the oracle: every routing border (INT8 units up to four rows, matrix-core tiles to eight, the
    one-pass kernel to 64, the many-row kernel beyond; the shapes each of them leaves to the plain kernels).  Bars: 1e-4 of the
    largest output of each activation row up to 64 rows (of the whole output where a row has fewer than 32 outputs to take a
    scale from), 2e-3 of the largest output beyond (the normalisation of GgufChecks.close, GgufChecks.java:110-120)."""
    from oracle import oracle
    rng = np.random.default_rng(20262)
    fmts = ["Q4_K", "Q5_K", "Q6_K", "Q4_0", "Q4_1", "Q8_0", "Q5_1", "Q2_K", "Q5_0", "Q3_K"]
    for case in range(80):
        fmt = fmts[case % len(fmts)]
        kq = BLOCK[fmt][0]
        if case % 7 == 0:
            k = 256 * int(rng.integers(1, 17))
        elif case % 7 == 1:
            k = 256 * int(rng.integers(17, 64))
        else:
            k = kq * int(rng.integers(1, 8192 // kq + 1))
        n = int(rng.integers(1, 700)) if case % 3 else int(rng.integers(1, 40))
        rows = int(rng.integers(1, 81))
        raw = random_valid_blocks(rng, fmt, n, k)
        w = weight(jn, fmt, raw, n, k)
        x = rng.standard_normal((rows, k)).astype(np.float32)
        if case % 4 == 0:
            x[rng.integers(0, rows)] *= np.float32(1e5)
        bias = rng.standard_normal(n).astype(np.float32) if case % 2 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k).astype(np.float64)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias) if bias is not None else None).numpy().astype(np.float64)
        if n >= 32 and rows <= 64:
            err = max(float(np.abs(y[r] - ref[r]).max()) / max(float(np.abs(ref[r]).max()), 1e-30) for r in range(rows))
        else:
            err = float(np.abs(y - ref).max()) / max(float(np.abs(ref).max()), 1e-30)
        assert err <= (MFMA_BAR if rows > 64 else GEMV_BAR), (case, fmt, n, k, rows, err)


@pytest.mark.parametrize("fmt", ["Q5_1", "Q2_K"])
@pytest.mark.parametrize("n,k", [(4, 256), (37, 1024), (259, 4096), (64, 14336), (6, 16384), (3, 512), (16, 320)])
def test_q5_1_q2_k_matrix_core_units(jn, fmt, n, k):
    """Q5_1 and Q2_K at one to four activation rows: the INT8 matrix-core kernel's units for them (rows of one to sixteen waves, a row
    count that is no multiple of four, with and without bias) and, for the shapes it does not take (fewer than four rows,
    rows of 320 values for Q5_1 only), the plain kernel - ordinary, outlier-ridden, tiny and unit-vector activations
    against the oracle, non-finite ones class by class."""
    from oracle import oracle
    if fmt == "Q2_K" and k % 256:
        pytest.skip("Q2_K rows are whole super-blocks")
    rng = np.random.default_rng(77 * GGML_ID[fmt] + n + k)
    raw = random_valid_blocks(rng, fmt, n, k)
    w = weight(jn, fmt, raw, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    xs = [rng.standard_normal(k).astype(np.float32)]
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, 5)] *= 1e4
    xs.append(x)
    xs.append((rng.standard_normal(k) * 1e-30).astype(np.float32))
    x = np.zeros(k, dtype=np.float32)
    x[k - 1] = 1.0
    xs.append(x)
    for i, x in enumerate(xs):
        b = bias if i % 2 == 0 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x[None, :], raw, b, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x[None, :]), w, jn.Tensor.of(b) if b is not None else None).numpy()
        assert norm_err(y, ref) <= GEMV_BAR, (fmt, n, k, i, norm_err(y, ref))
    x = rng.standard_normal(k).astype(np.float32)
    x[k // 3] = np.inf
    x[k // 2] = np.nan if n % 2 else -np.inf
    ref = oracle.gguf_linear(GGML_ID[fmt], x[None, :], raw, None, n, k)
    y = jn.Gguf.linear(jn.Tensor.of(x[None, :]), w, None).numpy()
    assert np.array_equal(np.isnan(y), np.isnan(ref)) and np.array_equal(np.isposinf(y), np.isposinf(ref)) and \
        np.array_equal(np.isneginf(y), np.isneginf(ref)), (fmt, n, k)
    for rows in (2, 3, 4):  # the same kernel with the activations of several rows in registers (rows of at most 4096 values)
        x = rng.standard_normal((rows, k)).astype(np.float32)
        x[rows - 1] *= 1e-3
        b = bias if rows % 2 else None
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, b, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(b) if b is not None else None).numpy()
        for r in range(rows):
            assert norm_err(y[r], ref[r]) <= GEMV_BAR, (fmt, n, k, rows, r, norm_err(y[r], ref[r]))


@pytest.mark.parametrize("fmt", sorted(REWRITTEN))
def test_rewritten_formats_keep_their_face_and_every_value(jn, fmt):
    """An uploaded Q5_0 / Q3_K weight reports the caller's format and byte count, dequantises to the oracle's bits for
    every bit pattern of quants and scales (all 256 byte values occur in random blocks; scales at both ends of their
    range), and multiplies like the format it was rewritten into holding the same values."""
    import ctypes as C
    from jitnn_amd import _lib as lib
    from oracle import oracle
    rng = np.random.default_rng(GGML_ID[fmt])
    n, k = 64, 2048
    raw = random_valid_blocks(rng, fmt, n, k, lo=1e-4, hi=2.0)
    w = weight(jn, fmt, raw, n, k)
    f, nn, kk, nb = C.c_int(), C.c_int(), C.c_int(), C.c_longlong()
    lib.check(lib.lib.jitnn_hip_weight_info(w.handle, C.byref(f), C.byref(nn), C.byref(kk), C.byref(nb)), "info")
    assert (f.value, nn.value, kk.value, nb.value) == (GGML_ID[fmt], n, k, raw.size)
    vals = oracle.dequantize(GGML_ID[fmt], raw, n * k)
    assert np.array_equal(bits(w.to_float_array()), bits(vals))
    x = rng.standard_normal((5, k)).astype(np.float32)
    y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
    ref = (x.astype(np.float64) @ vals.reshape(n, k).astype(np.float64).T)
    assert norm_err(y, ref) <= GEMV_BAR


def test_counters_follow_the_reference_byte_convention(jn):
    """Telemetry.tensorBytes (jitnn-core/src/main/java/ai/beestream/jitnn/engine/Telemetry.java:222-240): every input and output tensor once, block tensors at
    numel / blockValues * blockBytes."""
    rng = np.random.default_rng(8)
    n, k = 96, 512
    raw = random_valid_blocks(rng, "Q4_K", n, k)
    w = weight(jn, "Q4_K", raw, n, k)
    jn.stats_reset()
    jn.Gguf.linear(jn.Tensor.of(rng.standard_normal((3, k)).astype(np.float32)), w, jn.Tensor.of(np.zeros(n, dtype=np.float32)))
    jn.Gguf.linear(jn.Tensor.of(rng.standard_normal((70, k)).astype(np.float32)), w, None)
    jn.Gguf.dequantize(w)
    st = jn.stats()
    wb = n * k // 256 * 144
    assert st["linear_gemv"] == (1, wb + 4 * 3 * (k + n) + 4 * n)
    assert st["linear_mfma"] == (1, wb + 4 * 70 * (k + n))
    assert st["dequantize"] == (1, wb + 4 * n * k)
    assert st["llama_decode"] == (0, 0)
