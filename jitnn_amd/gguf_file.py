"""Host mirror of the reference's GgufFile (jitnn-gguf/src/main/java/ai/beestream/jitnn/gguf/GgufFile.java) over the
native reader (jitnn_hip_gguf_*): metadata, tensor listing in jitNN's axis order, raw bytes, and tensors - the
block-quantised ones go from the mapped file to HBM unchanged."""
from __future__ import annotations

import ctypes as C
import json
from dataclasses import dataclass

import numpy as np

from . import _lib
from .dtype import DType
from .tensor import Tensor

GGML_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K", 11: "Q3_K", 12: "Q4_K",
              13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 24: "I8", 25: "I16", 26: "I32", 27: "I64", 28: "F64", 30: "BF16"}


@dataclass(frozen=True)
class GgufTensorInfo:
    """gguf/GgufTensorInfo.java:29-39"""
    name: str
    shape: tuple
    type_id: int
    type: str | None   # ggml type name, None for an id this reader does not know
    offset: int
    bytes: int         # -1 when the type is unknown

    def numel(self) -> int:
        return int(np.prod(self.shape)) if self.shape else 1


class GgufFile:
    def __init__(self, handle, path):
        self._h, self._path = handle, str(path)
        v, a, off, nt, nkv = C.c_int(), C.c_int(), C.c_longlong(), C.c_longlong(), C.c_longlong()
        _lib.check(_lib.lib.jitnn_hip_gguf_header(handle, C.byref(v), C.byref(a), C.byref(off), C.byref(nt), C.byref(nkv)), "jitnn_hip_gguf_header")
        self._version, self._alignment, self._data_offset = v.value, a.value, off.value
        n = _lib.lib.jitnn_hip_gguf_metadata_json(handle, None, 0)
        buf = C.create_string_buffer(n + 1)
        _lib.lib.jitnn_hip_gguf_metadata_json(handle, buf, n + 1)
        self._metadata = json.loads(buf.value.decode("utf-8"))
        self._infos = {}
        name = C.create_string_buffer(1024)
        for i in range(nt.value):
            _lib.check(_lib.lib.jitnn_hip_gguf_tensor_name(handle, i, name, 1024), "jitnn_hip_gguf_tensor_name")
            t, nd, dims, fo, nb = C.c_int(), C.c_int(), (C.c_longlong * 8)(), C.c_longlong(), C.c_longlong()
            _lib.check(_lib.lib.jitnn_hip_gguf_tensor_info(handle, name.value, C.byref(t), C.byref(nd), dims, C.byref(fo), C.byref(nb)),
                       "jitnn_hip_gguf_tensor_info")
            nm = name.value.decode("utf-8")
            self._infos[nm] = GgufTensorInfo(nm, tuple(dims[j] for j in range(nd.value)), t.value, GGML_NAMES.get(t.value), fo.value, nb.value)

    @staticmethod
    def open(path) -> "GgufFile":
        """Reads the metadata and the tensor list; raises OSError for anything that is not a valid GGUF v2/v3 file."""
        h = C.c_void_p()
        _lib.check(_lib.lib.jitnn_hip_gguf_open(str(path).encode("utf-8"), C.byref(h)), "jitnn_hip_gguf_open")
        return GgufFile(h, path)

    def close(self):
        if self._h:
            _lib.lib.jitnn_hip_gguf_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- file
    def path(self): return self._path
    def version(self): return self._version
    def alignment(self): return self._alignment
    def data_offset(self): return self._data_offset

    # ---- metadata (gguf/GgufFile.java:203-316)
    def metadata(self): return self._metadata
    def keys(self): return list(self._metadata)
    def has(self, key): return key in self._metadata
    def get(self, key): return self._metadata.get(key)
    def architecture(self):
        v = self._metadata.get("general.architecture")
        return v if isinstance(v, str) else None

    def _required(self, key, types, what):
        if key not in self._metadata:
            raise ValueError(f"{self._path}: no metadata key {key}")
        v = self._metadata[key]
        if isinstance(v, bool) and bool not in types or not isinstance(v, types):
            raise ValueError(f"{key} is {type(v).__name__}, not {what}")
        return v

    def string(self, key): return self._required(key, (str,), "String")
    def bool(self, key): return self._required(key, (bool,), "Boolean")

    def long_value(self, key):
        return self._required(key, (int,), "an integer")

    def integer(self, key, fallback=None):
        if fallback is not None and not self.has(key):
            return fallback
        v = self.long_value(key)
        if not -(1 << 31) <= v < (1 << 31):
            raise ValueError(f"{key} = {v} is not an int")
        return v

    def float_value(self, key, fallback=None):
        if fallback is not None and not self.has(key):
            return fallback
        return float(np.float32(self._required(key, (int, float), "a number")))

    def strings(self, key):
        v = self._required(key, (list,), "String[]")
        if not all(isinstance(e, str) for e in v):
            raise ValueError(f"{key} is not an array of strings")
        return v

    def _numbers(self, key, what, lo=None, hi=None, integral=True):
        v = self._required(key, (list,), what)
        ok = (int,) if integral else (int, float)
        if not all(isinstance(e, ok) and not isinstance(e, bool) for e in v):
            raise ValueError(f"{key} is not {what}")
        if lo is not None and not all(lo <= e < hi for e in v):
            raise ValueError(f"{key} holds values outside {what}")
        return v

    def ints(self, key): return np.asarray(self._numbers(key, "int[]", -(1 << 31), 1 << 31), dtype=np.int32)
    def longs(self, key): return np.asarray(self._numbers(key, "long[]", -(1 << 63), 1 << 63), dtype=np.int64)
    def floats(self, key): return np.asarray(self._numbers(key, "float[]", integral=False), dtype=np.float32)

    # ---- tensors (gguf/GgufFile.java:309-366)
    def tensor_infos(self): return self._infos
    def has_tensor(self, name): return name in self._infos

    def info(self, name) -> GgufTensorInfo:
        if name not in self._infos:
            raise ValueError(f"{self._path}: no tensor {name}")
        return self._infos[name]

    def raw(self, name) -> np.ndarray:
        t = self.info(name)
        if t.bytes < 0:
            raise _lib.UnsupportedTypeError(f"{name}: ggml type {t.type_id} is unknown, so its size is too")
        out = np.empty(t.bytes, dtype=np.uint8)
        _lib.check(_lib.lib.jitnn_hip_gguf_tensor_read(self._h, name.encode("utf-8"), out.ctypes.data_as(C.c_void_p), t.bytes), "jitnn_hip_gguf_tensor_read")
        return out

    def tensor(self, name) -> Tensor:
        """Block-quantised types of the path become device-resident weights (raw blocks, unchanged); F32 loads as a host
        tensor; anything else has no tensor type here."""
        t = self.info(name)
        if t.type == "F32":
            return Tensor.of(self.raw(name).view(np.float32).reshape(t.shape))
        if t.type == "I32":
            return Tensor(t.shape, DType.I32, host=self.raw(name).view(np.int32).reshape(t.shape))
        if t.type in DType.__members__ and DType[t.type].is_block_quantized():
            _lib.init()
            h = C.c_void_p()
            _lib.check(_lib.lib.jitnn_hip_gguf_tensor_upload(self._h, name.encode("utf-8"), C.byref(h)), "jitnn_hip_gguf_tensor_upload")
            return Tensor(t.shape, DType[t.type], handle=h)
        raise _lib.UnsupportedTypeError(f"{name}: ggml type {t.type or 'id ' + str(t.type_id)} has no tensor type on this path")

    def tensors(self) -> dict:
        """Every tensor of the file by name; raises UnsupportedTypeError at the first one without a tensor type."""
        return {name: self.tensor(name) for name in self._infos}
