"""The synthetic-weight quantisers (quantizers.py at the repository root) produce valid blocks whose dequantisation (by the
oracle) is close to the input: checks layout packing against the pinned dequantisers."""
import numpy as np
import pytest
import torch

import quantizers
from helpers import BLOCK, GGML_ID
from oracle import oracle

# worst-case relative step of each format on N(0, sigma) rows (fraction of the block's range)
BAR = {"Q8_0": 1 / 127, "Q4_0": 1 / 7.0, "Q4_1": 1 / 14.0, "Q4_K": 1 / 12.0, "Q5_K": 1 / 26.0, "Q6_K": 1 / 28.0}


@pytest.mark.parametrize("fmt", ["Q8_0", "Q4_0", "Q4_1", "Q4_K", "Q5_K", "Q6_K"])
def test_roundtrip(fmt):
    g = torch.Generator().manual_seed(3)
    n, k = 16, 1024
    w = torch.randn(n, k, generator=g) * 0.02
    w[0, :256] = 0          # all-zero blocks
    w[1, :256] = 0.01       # constant blocks
    w[2, :256] = -w[2, :256].abs()  # all-negative
    raw = quantizers.quantize(fmt, w).numpy()
    qk, nb = BLOCK[fmt]
    assert raw.dtype == np.uint8 and raw.size == n * k // qk * nb
    d = oracle.dequantize(GGML_ID[fmt], raw, n * k).reshape(n, k)
    assert np.all(np.isfinite(d))
    x = w.numpy()
    blocks = x.reshape(-1, qk)
    rng_ = np.maximum(blocks.max(axis=1) - np.minimum(blocks.min(axis=1), 0), np.abs(blocks).max(axis=1))
    err = np.abs(d.reshape(-1, qk) - blocks).max(axis=1)
    assert np.all(err <= rng_ * BAR[fmt] + 1e-7), (fmt, float((err / (rng_ + 1e-12)).max()))
    assert np.abs(d[0, :256]).max() == 0


def test_q8_0_matches_oracle_bytes():
    g = torch.Generator().manual_seed(4)
    w = torch.randn(8, 256, generator=g)
    assert np.array_equal(quantizers.quantize_q8_0(w).numpy(), oracle.quantize_q8_0(w.numpy()))
