"""The operator API of the path, by the reference's names: Gguf.linear / Gguf.dequantize
(core/ops/Gguf.java:68-98), Quant.linear / Quant.quantize_q8 / Quant.dequantize (core/ops/Quant.java:42-80)
and the F facade (core/F.java:1039-1051).  Argument meaning and misuse errors follow the reference; the
arithmetic runs in libjitnn_hip.so."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .dtype import DType
from .tensor import Tensor


def _f32(x: Tensor, what: str) -> None:
    if x.dtype() != DType.F32:  # Checks.f32
        raise ValueError(f"{what} needs an FP32 input, got {x.dtype().name}")


def _linear(x: Tensor, w: Tensor, bias: Tensor | None, what: str) -> Tensor:
    if w.rank() != 2 or x.rank() < 1 or x.dim(-1) != w.dim(1):
        raise ValueError(f"{what}: input {list(x.shape())} and weight {list(w.shape())}")
    n, k = w.dim(0), w.dim(1)
    rows = x.numel() // k
    if bias is not None:
        _f32(bias, what)
        if bias.numel() != n:
            raise ValueError(f"{what}: bias {list(bias.shape())} for {n} outputs")
    xa = np.ascontiguousarray(x.numpy(), dtype=np.float32)
    ba = None if bias is None else np.ascontiguousarray(bias.numpy(), dtype=np.float32)
    y = np.empty(x.shape()[:-1] + (n,), dtype=np.float32)
    if rows > 0:
        _lib.check(_lib.lib.jitnn_hip_linear(w.handle, xa.ctypes.data_as(C.c_void_p), rows,
                                             None if ba is None else ba.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p)),
                   "jitnn_hip_linear")
    return Tensor.of(y)


class Quant:
    """Q8_0 quantisation, dequantisation and linear layers on Q8_0 weights (core/ops/Quant.java)."""

    @staticmethod
    def quantize_q8(x: Tensor) -> Tensor:
        _f32(x, "quantizeQ8")
        if x.rank() == 0 or x.dim(-1) % 32 != 0:
            raise ValueError(f"Q8_0 needs a last axis that is a multiple of 32, got {list(x.shape())}")
        xa = np.ascontiguousarray(x.numpy(), dtype=np.float32)
        q = np.empty(xa.size // 32 * 34, dtype=np.uint8)
        _lib.init()
        _lib.check(_lib.lib.jitnn_hip_quantize_q8_0(xa.ctypes.data_as(C.c_void_p), xa.size, q.ctypes.data_as(C.c_void_p)),
                   "jitnn_hip_quantize_q8_0")
        return Tensor.quantized(DType.Q8_0, q, *x.shape())

    @staticmethod
    def dequantize(q: Tensor) -> Tensor:
        if q.dtype() != DType.Q8_0:
            raise ValueError(f"dequantize needs a Q8_0 tensor, got {q.dtype().name}")
        return Tensor.of(q.to_float_array(), *q.shape())

    @staticmethod
    def linear(x: Tensor, w: Tensor, bias: Tensor | None = None) -> Tensor:
        _f32(x, "Q8_0 linear")
        if w.dtype() != DType.Q8_0:
            raise ValueError(f"Q8_0 linear: input {list(x.shape())} and weight {list(w.shape())} {w.dtype().name}")
        return _linear(x, w, bias, "Q8_0 linear")


class Gguf:
    """Linear layers and dequantisation for weights in GGUF block formats (core/ops/Gguf.java)."""

    @staticmethod
    def dequantize(w: Tensor) -> Tensor:
        if not w.dtype().is_block_quantized() or w.dtype() == DType.Q8_0:
            raise ValueError(f"not a GGUF format with jitNN dequantisation: {w.dtype().name}")
        return Tensor.of(w.to_float_array(), *w.shape())

    @staticmethod
    def linear(x: Tensor, w: Tensor, bias: Tensor | None = None) -> Tensor:
        """y = x W^T + b, W [N, K] in a GGUF format, x FP32 [..., K]; b may be None."""
        _f32(x, "linear")
        if w.dtype() == DType.Q8_0:
            return Quant.linear(x, w, bias)
        if not w.dtype().is_block_quantized():
            raise ValueError(f"not a GGUF block format: {w.dtype().name}")
        return _linear(x, w, bias, f"{w.dtype().name} linear")


class F:
    """The functional facade's entries for this path (core/F.java:1039-1051)."""

    quantize_q8 = staticmethod(Quant.quantize_q8)
    dequantize = staticmethod(Quant.dequantize)
    linear_q8 = staticmethod(Quant.linear)
