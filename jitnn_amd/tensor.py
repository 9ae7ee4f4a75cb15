"""Host-side tensors of the path: FP32 activations in host memory (numpy), block-quantised weights
resident in HBM behind a native handle.  Mirrors the part of the reference's Tensor API the path uses
(core/Tensor.java:249-278 quantized/persistent, :520-555 toFloatArray)."""
from __future__ import annotations

import ctypes as C
import weakref

import numpy as np

from . import _lib
from .dtype import DType


class Tensor:
    def __init__(self, shape, dtype: DType, host: np.ndarray | None = None, handle=None):
        self._shape = tuple(int(d) for d in shape)
        self._dtype = dtype
        self._host = host
        self._handle = handle
        if handle is not None:
            self._finalizer = weakref.finalize(self, _lib.lib.jitnn_hip_weight_free, handle)

    # ---- construction
    @staticmethod
    def of(values, *dims) -> "Tensor":
        """FP32 tensor from host values (Tensor.of)."""
        a = np.ascontiguousarray(values, dtype=np.float32)
        if dims:
            if int(np.prod(dims)) != a.size:
                raise ValueError(f"{a.size} values do not fill shape {list(dims)}")
            a = a.reshape(dims)
        return Tensor(a.shape, DType.F32, host=a)

    @staticmethod
    def quantized(dtype: DType, blocks, *dims) -> "Tensor":
        """A weight in a GGUF block format from its raw blocks (Tensor.quantized, core/Tensor.java:249-251):
        persistent, uploaded once, kept byte for byte in HBM.  The last axis must be a multiple of the block size
        and the byte count must match (core/Tensor.java:266-276)."""
        if not dtype.is_block_quantized():
            raise ValueError(f"{dtype.name} is not a block-quantised type")
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        if len(dims) == 0 or dims[-1] % dtype.block_values() != 0:
            raise ValueError(f"{dtype.name} weight of shape {list(dims)}: last axis not a multiple of its block of {dtype.block_values()}")
        raw = np.ascontiguousarray(np.frombuffer(blocks, dtype=np.uint8) if isinstance(blocks, (bytes, bytearray, memoryview)) else blocks,
                                   dtype=np.uint8).reshape(-1)
        numel = int(np.prod(dims))
        expected = numel // dtype.block_values() * dtype.block_bytes()
        if raw.size != expected:
            raise ValueError(f"{dtype.name} tensor of shape {list(dims)} needs {expected} array elements, got {raw.size}")
        k = dims[-1]
        n = numel // k
        _lib.init()
        h = C.c_void_p()
        _lib.check(_lib.lib.jitnn_hip_weight_upload(dtype.ggml_id, raw.ctypes.data_as(C.c_void_p), raw.size, n, k, C.byref(h)),
                   "jitnn_hip_weight_upload")
        return Tensor(dims, dtype, handle=h)

    # ---- accessors
    def dtype(self) -> DType:
        return self._dtype

    def shape(self) -> tuple:
        return self._shape

    def rank(self) -> int:
        return len(self._shape)

    def dim(self, i: int) -> int:
        return self._shape[i]

    def numel(self) -> int:
        return int(np.prod(self._shape)) if self._shape else 1

    def reshape(self, *dims) -> "Tensor":
        if self._dtype != DType.F32:
            raise ValueError("only FP32 tensors reshape on this path")
        return Tensor.of(self._host.reshape(dims))

    @property
    def handle(self):
        return self._handle

    def numpy(self) -> np.ndarray:
        if self._dtype != DType.F32:
            raise ValueError("numpy() is for FP32 tensors; use to_float_array() to dequantise")
        return self._host

    def to_int_array(self) -> np.ndarray:
        """Row-major values of an I32 tensor (Tensor.toIntArray)."""
        if self._dtype != DType.I32:
            raise ValueError(f"to_int_array() on a {self._dtype.name} tensor")
        return self._host.reshape(-1).copy()

    def to_float_array(self) -> np.ndarray:
        """Row-major values as FP32; block tensors are dequantised on the device, bit-identical to the reference's
        per-value decode (Tensor.toFloatArray, core/Tensor.java:539-555)."""
        if self._dtype == DType.F32:
            return self._host.reshape(-1).copy()
        if self._dtype == DType.I32:
            return self._host.reshape(-1).astype(np.float32)
        y = np.empty(self.numel(), dtype=np.float32)
        _lib.check(_lib.lib.jitnn_hip_dequantize(self._handle, y.ctypes.data_as(C.c_void_p)), "jitnn_hip_dequantize")
        return y
