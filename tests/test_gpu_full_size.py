"""The BASELINE configurations at their full sizes.  The oracle is a scalar FP64 loop (a third of a second per 58 M
weights and activation row), so at these sizes the whole matrix is checked through properties that do not depend on
the size - linearity in x, unit vectors give columns of the dequantised matrix, a batch agrees with its rows taken
one at a time, the many-row path agrees with the GEMV path - and directly against the oracle on a sample of rows
and, for the dequantiser, bit by bit on the whole 58 M-value matrix."""
import numpy as np
import pytest

from helpers import BLOCK, GGML_ID, norm_err, random_valid_blocks

pytestmark = pytest.mark.gpu

CONFIGS = [  # (format, n, k, batch sizes): BASELINE configs 1-4, and the 16 / 40 / 64 rows bench.py times on configs 1-3's matrices
    ("Q8_0", 4096, 4096, (1, 40)),
    ("Q4_0", 11008, 4096, (1, 4, 40)),
    ("Q4_K", 14336, 4096, (1, 2, 8, 16, 40, 64)),
    ("Q6_K", 128256, 4096, (1,)),
    # the other weights of a Q4_K_M / Q5_K_M layer at the row counts of a short prompt: ffn_down (long rows: the one-pass
    # kernel from three rows on, two tiles per wave from 17) and a Q5_K gate
    ("Q6_K", 4096, 14336, (1, 5, 40)),
    ("Q5_K", 14336, 4096, (1, 16, 64)),
]


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


def rows_of(raw, fmt, k, sel):
    qk, nb = BLOCK[fmt]
    rb = k // qk * nb
    return np.ascontiguousarray(raw.reshape(-1, rb)[sel]).reshape(-1)


def baseline_weight(fmt, n, k, seed):
    """The BASELINE configurations' weight: FP32 [n, k] drawn from N(0, 0.02) and quantised to fmt - Q8_0 with the
    reference's own quantiser as the oracle restates it (Quant.java:102-118), the others with quantizers.py; drawn
    and quantised on the GPU by torch in row chunks (set-up only: the bytes then go to the oracle and the library)."""
    import torch

    import quantizers
    from oracle import oracle
    g = torch.Generator(device="cuda").manual_seed(seed)
    parts = []
    for r0 in range(0, n, 8192):
        w = torch.randn(min(8192, n - r0), k, generator=g, device="cuda") * 0.02
        parts.append(oracle.quantize_q8_0(w.cpu().numpy()) if fmt == "Q8_0" else quantizers.quantize(fmt, w).cpu().numpy())
        del w
    torch.cuda.empty_cache()
    return np.concatenate(parts)


@pytest.mark.parametrize("source", ["random_blocks", "normal_0.02_quantised"])
@pytest.mark.parametrize("fmt,n,k,batches", CONFIGS)
def test_full_size_gemv(jn, fmt, n, k, batches, source):
    from oracle import oracle
    rng = np.random.default_rng(GGML_ID[fmt] * 7 + n)
    raw = random_valid_blocks(rng, fmt, n, k) if source == "random_blocks" else baseline_weight(fmt, n, k, 1000 + GGML_ID[fmt])
    w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
    sel = np.unique(rng.integers(0, n, size=48))
    sub = rows_of(raw, fmt, k, sel)
    bmax = max(batches)
    x = rng.standard_normal((bmax, k)).astype(np.float32)
    singles = np.stack([jn.Gguf.linear(jn.Tensor.of(x[r:r + 1]), w, None).numpy()[0] for r in range(bmax)])
    for b in batches:
        y = jn.Gguf.linear(jn.Tensor.of(x[:b]), w, None).numpy()
        assert y.shape == (b, n)
        # a sample of rows of the full matrix against the oracle
        ref = oracle.gguf_linear(GGML_ID[fmt], x[:b], sub, None, len(sel), k)
        assert norm_err(y[:, sel], ref) <= 1e-4, (fmt, b, norm_err(y[:, sel], ref))
        # every row of the batch against the same row on its own (other kernels for other batch sizes)
        assert norm_err(y, singles[:b]) <= 1e-4, (fmt, b)
    # linearity over the whole matrix: W (a x0 + c x1) = a W x0 + c W x1
    x0, x1 = x[0], rng.standard_normal(k).astype(np.float32)
    a, c = np.float32(0.75), np.float32(-1.5)
    y1 = jn.Gguf.linear(jn.Tensor.of(x1[None]), w, None).numpy()[0]
    ymix = jn.Gguf.linear(jn.Tensor.of((a * x0 + c * x1)[None]), w, None).numpy()[0]
    lin = a * singles[0].astype(np.float64) + c * y1.astype(np.float64)
    assert norm_err(ymix, lin) <= 1e-4, fmt
    # a unit vector picks a column of the dequantised matrix (checked on the sampled rows, against the oracle's dequantiser)
    j = int(rng.integers(0, k))
    e = np.zeros((1, k), dtype=np.float32)
    e[0, j] = 1.0
    col = jn.Gguf.linear(jn.Tensor.of(e), w, None).numpy()[0]
    deq = oracle.dequantize(GGML_ID[fmt], sub, len(sel) * k).reshape(len(sel), k)
    assert np.allclose(col[sel], deq[:, j], rtol=2e-6, atol=1e-7), fmt


def test_full_size_dequantize_bit_exact(jn):
    """Config 3's matrix, all 58.7 M values, bit for bit against the oracle's dequantiser."""
    from oracle import oracle
    n, k = 14336, 4096
    rng = np.random.default_rng(31)
    raw = random_valid_blocks(rng, "Q4_K", n, k)
    got = jn.Gguf.dequantize(jn.Tensor.quantized(jn.DType.Q4_K, raw, n, k)).numpy().reshape(-1)
    ref = oracle.dequantize(GGML_ID["Q4_K"], raw, n * k)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("fmt,n,k", [("Q4_K", 14336, 4096), ("Q6_K", 4096, 14336), ("Q4_K", 4096, 4096)])
def test_full_size_prefill_512(jn, fmt, n, k):
    """The 512-token linears of config 5 on the matrix-core path: a sample of weight rows against the oracle on every
    token, and the first 8 tokens against the FP32-grade GEMV path over the whole matrix."""
    from oracle import oracle
    rng = np.random.default_rng(n + k)
    raw = random_valid_blocks(rng, fmt, n, k)
    w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
    x = rng.standard_normal((512, k)).astype(np.float32)
    y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
    assert y.shape == (512, n)
    sel = np.unique(rng.integers(0, n, size=12))
    ref = oracle.gguf_linear(GGML_ID[fmt], x, rows_of(raw, fmt, k, sel), None, len(sel), k)
    assert norm_err(y[:, sel], ref) <= 2e-3, (fmt, norm_err(y[:, sel], ref))
    y8 = jn.Gguf.linear(jn.Tensor.of(x[:8]), w, None).numpy()
    assert norm_err(y[:8], y8) <= 2e-3, fmt
