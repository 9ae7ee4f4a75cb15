"""FP32 -> GGUF block quantisers for synthetic test and benchmark weights (torch ops: CPU or GPU tensors).

Test and benchmark tooling (it sits beside bench.py, which draws its weights with it; tests/ imports it too), not part of
the path: the reference has no quantiser for these formats besides Q8_0
(core/ops/Quant.java:86-119), and parity is defined on the bytes both sides consume.  The layouts are ggml's
block_q4_0 ... block_q6_K; the rounding choices are simple min/max fits, not ggml's error-minimising
searches.  Every function returns a flat uint8 tensor of n*k/qk*nb bytes for w [n, k].
"""
from __future__ import annotations

import torch


def _f16_bytes(v: torch.Tensor) -> torch.Tensor:
    """float tensor [...] -> uint8 [..., 2] little-endian binary16 (round to nearest even)."""
    return v.to(torch.float16).contiguous().view(torch.uint8).reshape(*v.shape, 2)


def _f16_round(v: torch.Tensor) -> torch.Tensor:
    return v.to(torch.float16).to(torch.float32)


def quantize_q4_0(w: torch.Tensor) -> torch.Tensor:
    x = w.float().reshape(-1, 32)
    idx = x.abs().argmax(dim=1, keepdim=True)
    mx = x.gather(1, idx)
    d = mx / -8.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    q = torch.clamp((x * inv + 8.5).floor(), 0, 15).to(torch.uint8)
    qs = q[:, :16] | (q[:, 16:] << 4)
    return torch.cat([_f16_bytes(d[:, 0]), qs], dim=1).reshape(-1)


def quantize_q4_1(w: torch.Tensor) -> torch.Tensor:
    x = w.float().reshape(-1, 32)
    mn = x.min(dim=1, keepdim=True).values
    mx = x.max(dim=1, keepdim=True).values
    d = (mx - mn) / 15.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    q = torch.clamp(((x - mn) * inv + 0.5).floor(), 0, 15).to(torch.uint8)
    qs = q[:, :16] | (q[:, 16:] << 4)
    return torch.cat([_f16_bytes(d[:, 0]), _f16_bytes(mn[:, 0]), qs], dim=1).reshape(-1)


def _k_scales(x: torch.Tensor, levels: int):
    """x [nb, 8, 32] -> (d16, dmin16 [nb], sc, mn [nb, 8] ints 0..63) for value = d*sc*q - dmin*mn, q in 0..levels."""
    lo = torch.clamp(x.min(dim=2).values, max=0.0)
    hi = torch.clamp(x.max(dim=2).values, min=0.0)
    scale = (hi - lo) / levels
    mins = -lo
    d = scale.max(dim=1, keepdim=True).values / 63.0
    dmin = mins.max(dim=1, keepdim=True).values / 63.0
    sc = torch.where(d > 0, (scale / d.clamp_min(1e-30)).round(), torch.zeros_like(scale)).clamp(0, 63)
    mn = torch.where(dmin > 0, (mins / dmin.clamp_min(1e-30)).round(), torch.zeros_like(mins)).clamp(0, 63)
    return d[:, 0], dmin[:, 0], sc.to(torch.int32), mn.to(torch.int32)


def _pack_k_scales(sc: torch.Tensor, mn: torch.Tensor) -> torch.Tensor:
    """Inverse of ggml's get_scale_min_k4: [nb, 8] x2 -> uint8 [nb, 12]."""
    s = torch.zeros(sc.shape[0], 12, dtype=torch.int32, device=sc.device)
    s[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    s[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
    s[:, 8:12] = (sc[:, 4:8] & 15) | ((mn[:, 4:8] & 15) << 4)
    return s.to(torch.uint8)


def _quantize_k45(w: torch.Tensor, levels: int):
    x = w.float().reshape(-1, 8, 32)
    d, dmin, sc, mn = _k_scales(x, levels)
    dh, dminh = _f16_round(d), _f16_round(dmin)
    step = (dh[:, None] * sc.float())[:, :, None]
    off = (dminh[:, None] * mn.float())[:, :, None]
    q = torch.where(step > 0, ((x + off) / step.clamp_min(1e-30)).round(), torch.zeros_like(x)).clamp(0, levels).to(torch.int32)
    return d, dmin, sc, mn, q


def quantize_q4_k(w: torch.Tensor) -> torch.Tensor:
    d, dmin, sc, mn, q = _quantize_k45(w, 15)
    q = q.reshape(-1, 4, 2, 32)
    qs = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).to(torch.uint8).reshape(-1, 128)
    return torch.cat([_f16_bytes(d), _f16_bytes(dmin), _pack_k_scales(sc, mn), qs], dim=1).reshape(-1)


def quantize_q5_k(w: torch.Tensor) -> torch.Tensor:
    d, dmin, sc, mn, q = _quantize_k45(w, 31)
    q = q.reshape(-1, 8, 32)
    low = (q & 15).reshape(-1, 4, 2, 32)
    qs = (low[:, :, 0, :] | (low[:, :, 1, :] << 4)).to(torch.uint8).reshape(-1, 128)
    hb = (q >> 4)  # [nb, 8, 32]: bit sub of qh[l]
    shifts = torch.arange(8, device=q.device, dtype=torch.int32).reshape(1, 8, 1)
    qh = (hb << shifts).sum(dim=1).to(torch.uint8)
    return torch.cat([_f16_bytes(d), _f16_bytes(dmin), _pack_k_scales(sc, mn), qh, qs], dim=1).reshape(-1)


def quantize_q6_k(w: torch.Tensor) -> torch.Tensor:
    x = w.float().reshape(-1, 16, 16)  # [nb, group (8n + 2k + l/16), 16]
    idx = x.abs().argmax(dim=2, keepdim=True)
    mx = x.gather(2, idx)[:, :, 0]
    scale = mx / -32.0
    d = scale.abs().max(dim=1, keepdim=True).values / 127.0
    sc = torch.where(d > 0, (scale / d.clamp_min(1e-30)).round(), torch.zeros_like(scale)).clamp(-128, 127)
    dh = _f16_round(d[:, 0])
    step = (dh[:, None] * sc)[:, :, None]
    q = torch.where(step != 0, (x / torch.where(step != 0, step, torch.ones_like(step))).round(), torch.zeros_like(x)).clamp(-32, 31)
    q = (q + 32).to(torch.int32)  # 0..63
    # element e of the block: n=e/128, k=(e%128)/32, l=e%32; group index 8n + 2k + l/16, position l%16
    q = q.reshape(-1, 2, 4, 2, 16).reshape(-1, 2, 4, 32)  # [nb, n, k, l]
    low, high = q & 15, q >> 4
    ql = torch.stack([low[:, :, 0] | (low[:, :, 2] << 4), low[:, :, 1] | (low[:, :, 3] << 4)], dim=2)  # [nb, n, k%2, l]
    qh = high[:, :, 0] | (high[:, :, 1] << 2) | (high[:, :, 2] << 4) | (high[:, :, 3] << 6)                # [nb, n, l]
    sc8 = sc.to(torch.int8).view(torch.uint8)
    return torch.cat([ql.to(torch.uint8).reshape(-1, 128), qh.to(torch.uint8).reshape(-1, 64), sc8, _f16_bytes(d[:, 0])], dim=1).reshape(-1)


def quantize_q8_0(w: torch.Tensor) -> torch.Tensor:
    """The reference quantiser's arithmetic (core/ops/Quant.java:102-118) in torch; the product path for this
    format is jitnn_hip_quantize_q8_0, this one only serves CPU-side tests of the other tools."""
    x = w.double().reshape(-1, 32)
    amax = x.abs().max(dim=1, keepdim=True).values
    d = (amax / 127.0).float()
    s = torch.where(d > 0, x / d.double().clamp_min(1e-300), torch.zeros_like(x))
    q = (torch.sign(s) * (s.abs() + 0.5).floor()).clamp(-127, 127).to(torch.int8).view(torch.uint8)
    return torch.cat([_f16_bytes(d[:, 0]), q], dim=1).reshape(-1)


QUANTIZERS = {"Q4_0": quantize_q4_0, "Q4_1": quantize_q4_1, "Q4_K": quantize_q4_k, "Q5_K": quantize_q5_k, "Q6_K": quantize_q6_k,
              "Q8_0": quantize_q8_0}


def quantize(fmt: str, w: torch.Tensor, chunk_rows: int = 4096) -> torch.Tensor:
    """w [n, k] -> flat uint8 blocks, processed in row chunks to bound memory."""
    n = w.shape[0]
    parts = [QUANTIZERS[fmt](w[r:r + chunk_rows]) for r in range(0, n, chunk_rows)]
    return torch.cat(parts)
