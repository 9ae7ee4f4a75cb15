"""Vectorised numpy dequantisers written from ggml's published block definitions (block_q4_0 ...
block_q6_K: shifts and masks over whole blocks), independent of the per-element division/remainder
form the oracle restates.  Used (a) to cross-check the oracle on random bytes and (b) as a fast
expected-value generator at sizes where the scalar oracle would take minutes.

Arithmetic is strict binary32 in the reference's operation order, so results are comparable bit for bit.
"""
from __future__ import annotations

import numpy as np

f32 = np.float32


def _f16(b: np.ndarray) -> np.ndarray:
    """little-endian byte pairs [..., 2] -> float32"""
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)[..., 0]


def _scale_min_k4(s: np.ndarray):
    """ggml get_scale_min_k4 on scales [nb, 12] -> (sc [nb, 8], mn [nb, 8]) as ints."""
    s = s.astype(np.int32)
    sc = np.empty(s.shape[:-1] + (8,), dtype=np.int32)
    mn = np.empty_like(sc)
    sc[..., :4] = s[..., 0:4] & 63
    mn[..., :4] = s[..., 4:8] & 63
    sc[..., 4:] = (s[..., 8:12] & 0xF) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, mn


def dequant(fmt: str, raw: np.ndarray) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    if fmt == "Q8_0":
        b = raw.reshape(-1, 34)
        d = _f16(b[:, 0:2])
        q = b[:, 2:].view(np.int8).astype(f32)
        return (d[:, None] * q).reshape(-1)
    if fmt == "Q4_0":
        b = raw.reshape(-1, 18)
        d = _f16(b[:, 0:2])
        qs = b[:, 2:].astype(np.int32)
        q = np.concatenate([qs & 0xF, qs >> 4], axis=1) - 8
        return (q.astype(f32) * d[:, None]).reshape(-1)
    if fmt == "Q4_1":
        b = raw.reshape(-1, 20)
        d, m = _f16(b[:, 0:2]), _f16(b[:, 2:4])
        qs = b[:, 4:].astype(np.int32)
        q = np.concatenate([qs & 0xF, qs >> 4], axis=1)
        return (q.astype(f32) * d[:, None] + m[:, None]).reshape(-1)
    if fmt == "Q5_0":
        b = raw.reshape(-1, 22)
        d = _f16(b[:, 0:2])
        qh = b[:, 2:6].copy().view(np.uint32)[:, 0]
        qs = b[:, 6:].astype(np.int32)
        bits = ((qh[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(np.int32)
        q = np.concatenate([qs & 0xF, qs >> 4], axis=1) + 16 * bits - 16
        return (q.astype(f32) * d[:, None]).reshape(-1)
    if fmt == "Q5_1":
        b = raw.reshape(-1, 24)
        d, m = _f16(b[:, 0:2]), _f16(b[:, 2:4])
        qh = b[:, 4:8].copy().view(np.uint32)[:, 0]
        qs = b[:, 8:].astype(np.int32)
        bits = ((qh[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(np.int32)
        q = np.concatenate([qs & 0xF, qs >> 4], axis=1) + 16 * bits
        return (q.astype(f32) * d[:, None] + m[:, None]).reshape(-1)
    if fmt in ("Q4_K", "Q5_K"):
        nb = 144 if fmt == "Q4_K" else 176
        b = raw.reshape(-1, nb)
        d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
        sc, mn = _scale_min_k4(b[:, 4:16])
        qs = b[:, nb - 128:].astype(np.int32).reshape(-1, 4, 32)
        q = np.stack([qs & 0xF, qs >> 4], axis=2)  # [nb, 4, 2, 32] -> sub = 2j+half
        if fmt == "Q5_K":
            qh = b[:, 16:48].astype(np.int32)  # [nb, 32]
            sub = np.arange(8).reshape(1, 4, 2, 1)
            q = q + 16 * ((qh[:, None, None, :] >> sub) & 1)
        q = q.reshape(-1, 8, 32).astype(f32)
        a = (d[:, None] * sc.astype(f32))[:, :, None] * q
        m = (dmin[:, None] * mn.astype(f32))[:, :, None]
        return (a - m).reshape(-1)
    if fmt == "Q6_K":
        b = raw.reshape(-1, 210)
        ql = b[:, 0:128].astype(np.int32).reshape(-1, 2, 2, 32)    # [nb, n, k%2, l]
        qh = b[:, 128:192].astype(np.int32).reshape(-1, 2, 32)     # [nb, n, l]
        sc = b[:, 192:208].view(np.int8).astype(np.int32).reshape(-1, 2, 4, 2)  # idx 8n + 2k + l/16
        d = _f16(b[:, 208:210])
        low = np.stack([ql[:, :, 0] & 0xF, ql[:, :, 1] & 0xF, ql[:, :, 0] >> 4, ql[:, :, 1] >> 4], axis=2)  # [nb, n, k, l]
        hi = np.stack([(qh >> (2 * k)) & 3 for k in range(4)], axis=2)
        q = (low | (hi << 4)) - 32
        scl = np.repeat(sc, 16, axis=3)  # [nb, n, k, 32]
        a = d[:, None, None, None] * scl.astype(f32)
        return (a * q.astype(f32)).reshape(-1)
    if fmt == "Q2_K":
        b = raw.reshape(-1, 84)
        scales = b[:, 0:16].astype(np.int32).reshape(-1, 2, 4, 2)  # idx 8n + 2j + l/16
        qs = b[:, 16:80].astype(np.int32).reshape(-1, 2, 32)
        d, dmin = _f16(b[:, 80:82]), _f16(b[:, 82:84])
        q = np.stack([(qs >> (2 * j)) & 3 for j in range(4)], axis=2)  # [nb, n, j, l]
        scl = np.repeat(scales, 16, axis=3)
        a = (d[:, None, None, None] * (scl & 0xF).astype(f32)) * q.astype(f32)
        m = dmin[:, None, None, None] * (scl >> 4).astype(f32)
        return (a - m).reshape(-1)
    if fmt == "Q3_K":
        b = raw.reshape(-1, 110)
        hmask = b[:, 0:32].astype(np.int32)
        qs = b[:, 32:96].astype(np.int32).reshape(-1, 2, 32)
        s = b[:, 96:108].astype(np.int32)
        d = _f16(b[:, 108:110])
        idx = np.arange(16)
        low = np.where(idx < 8, s[:, idx % 8] & 0xF, s[:, idx % 8] >> 4)
        high = (s[:, 8 + idx % 4] >> (2 * (idx // 4))) & 3
        sc = (low | (high << 4)) - 32  # [nb, 16], index 8n + 2j + l/16
        q = np.stack([(qs >> (2 * j)) & 3 for j in range(4)], axis=2)  # [nb, n, j, l]
        bit = np.stack([np.stack([(hmask >> (4 * n + j)) & 1 for j in range(4)], axis=1) for n in range(2)], axis=1)
        q = q - np.where(bit == 1, 0, 4)
        scl = np.repeat(sc.reshape(-1, 2, 4, 2), 16, axis=3)
        return ((d[:, None, None, None] * scl.astype(f32)) * q.astype(f32)).reshape(-1)
    raise ValueError(fmt)
