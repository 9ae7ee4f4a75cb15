"""A minimal GGUF v3 writer for tests that need a model file of their own (no downloads): metadata of the common types
and tensors given as raw bytes.  Test infrastructure."""
from __future__ import annotations

import struct

import numpy as np

U32, I32, F32, BOOL, STR, ARR, U64 = 4, 5, 6, 7, 8, 9, 10


def _s(b: bytearray, s: str):
    e = s.encode("utf-8")
    b += struct.pack("<Q", len(e)) + e


def _value(b: bytearray, v):
    if isinstance(v, bool):
        b += struct.pack("<I?", BOOL, v)
    elif isinstance(v, int):
        b += struct.pack("<II", U32, v) if 0 <= v < (1 << 32) else struct.pack("<Ii", I32, v)
    elif isinstance(v, float):
        b += struct.pack("<If", F32, v)
    elif isinstance(v, str):
        b += struct.pack("<I", STR)
        _s(b, v)
    elif isinstance(v, (list, tuple)):
        first = v[0]
        et = STR if isinstance(first, str) else F32 if isinstance(first, float) else I32
        b += struct.pack("<IIQ", ARR, et, len(v))
        for e in v:
            if et == STR:
                _s(b, e)
            else:
                b += struct.pack("<f" if et == F32 else "<i", e)
    else:
        raise TypeError(type(v))


def write_gguf(path, metadata: dict, tensors: list, alignment: int = 32):
    """tensors: [(name, shape outermost-first, ggml type id, raw bytes as uint8 array)]."""
    b = bytearray(b"GGUF")
    b += struct.pack("<IQQ", 3, len(tensors), len(metadata))
    for k, v in metadata.items():
        _s(b, k)
        _value(b, v)
    off = 0
    offsets = []
    tensors = [(name, shape, tid, np.ascontiguousarray(raw).view(np.uint8).reshape(-1)) for name, shape, tid, raw in tensors]
    for name, shape, tid, raw in tensors:
        _s(b, name)
        b += struct.pack("<I", len(shape))
        for dim in reversed(shape):  # GGUF lists the innermost axis first
            b += struct.pack("<Q", dim)
        b += struct.pack("<IQ", tid, off)
        offsets.append(off)
        off += (len(raw) + alignment - 1) // alignment * alignment
    b += b"\0" * ((-len(b)) % alignment)
    for (name, shape, tid, raw), o in zip(tensors, offsets):
        data = raw.tobytes()
        b += data + b"\0" * ((-len(data)) % alignment)
    with open(path, "wb") as f:
        f.write(bytes(b))
