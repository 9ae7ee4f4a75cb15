"""Run in a fresh process by tests/test_gpu_knobs.py with ONE JITNN_HIP_* environment switch set (the library reads its
switches once, at jitnn_hip_init): a short slice of the parity checks on the code path that switch selects.
Prints "knob ok" and exits 0, or raises."""
import os
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from helpers import GGML_ID, norm_err, random_valid_blocks  # noqa: E402
from oracle import oracle  # noqa: E402


def linear_err(jn, fmt, n, k, rows, rng, bias=False):
    raw = random_valid_blocks(rng, fmt, n, k)
    w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32) if bias else None
    y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(b) if bias else None).numpy()
    return norm_err(y, oracle.gguf_linear(GGML_ID[fmt], x, raw, b, n, k))


def main(knob: str) -> None:
    assert knob in os.environ, knob
    import jitnn_amd as jn
    jn.init()
    rng = np.random.default_rng(len(knob))
    if knob == "JITNN_HIP_GEMV_MAX_ROWS":
        # =8: nine rows and more leave the FP32-grade GEMV range for the FP16 matrix-core path (bar 2e-3); up to eight stay (1e-4)
        assert os.environ[knob] == "8"
        for fmt in ("Q4_K", "Q6_K", "Q8_0"):
            assert linear_err(jn, fmt, 96, 1024, 8, rng) <= 1e-4
            e = linear_err(jn, fmt, 96, 1024, 40, rng, bias=True)
            assert 1e-6 < e <= 2e-3, (fmt, e)   # (an FP32-grade result would be below 1e-6: the switch did move the call)
    elif knob == "JITNN_HIP_GEMV_I8":
        # =0: batch-1 K-quant GEMV on the FP32 register kernels (rows of at most 4096 values) and the K-split kernel (longer rows)
        assert os.environ[knob] == "0"
        for fmt in ("Q4_K", "Q5_K", "Q6_K"):
            for n, k in ((257, 4096), (64, 14336), (5, 512)):
                assert linear_err(jn, fmt, n, k, 1, rng, bias=n == 64) <= 1e-4, (fmt, n, k)
    elif knob == "JITNN_HIP_TRANSCODE":
        # =0: uploaded Q5_0 / Q3_K blocks stay byte for byte as the file has them and run on the plain kernels
        assert os.environ[knob] == "0"
        for fmt in ("Q5_0", "Q3_K"):
            n, k = 48, 1024
            raw = random_valid_blocks(rng, fmt, n, k)
            w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
            deq = w.to_float_array()
            assert np.array_equal(deq.view(np.uint32), oracle.dequantize(GGML_ID[fmt], raw, n * k).view(np.uint32)), fmt
            for rows in (1, 5, 40, 96):
                x = rng.standard_normal((rows, k)).astype(np.float32)
                y = jn.Gguf.linear(jn.Tensor.of(x), w, None).numpy()
                assert norm_err(y, oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)) <= (1e-4 if rows <= 64 else 2e-3), (fmt, rows)
    else:
        raise SystemExit(f"unknown knob {knob}")
    print("knob ok", flush=True)


if __name__ == "__main__":
    main(sys.argv[1])
