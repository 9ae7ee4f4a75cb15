"""ctypes binding of libjitnn_hip.so (the C ABI in include/jitnn_hip.h).

The library is the only implementation of the path: if it is missing or cannot be loaded this module
raises, there is no other code path to fall back to.  It is built in-tree by jitnn_amd/csrc/Makefile
(see __graft_entry__.build).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libjitnn_hip.so"

OK, EINVAL, EDEVICE, ENODEVICE, ENOMEM, EIO, EUNSUPPORTED = 0, -1, -2, -3, -4, -5, -6


class UnsupportedTypeError(TypeError):
    """A ggml type this path has no tensor type for (the reference's UnsupportedOperationException)."""


class JitnnError(RuntimeError):
    """A native call failed (the reference's JitnnException, core/JitnnException.java:18-25)."""


def _bind() -> C.CDLL:
    if not LIB_PATH.exists():
        raise JitnnError(f"{LIB_PATH} is not built: run `make -C jitnn_amd/csrc` (or __graft_entry__.build())")
    lib = C.CDLL(str(LIB_PATH))
    vp, i, ll, fp = C.c_void_p, C.c_int, C.c_longlong, C.POINTER(C.c_float)
    sig = {
        "jitnn_hip_init": (i, [i]),
        "jitnn_hip_device_info": (i, [C.c_char_p, i, C.POINTER(i), C.POINTER(ll)]),
        "jitnn_hip_last_error": (C.c_char_p, []),
        "jitnn_hip_sync": (i, []),
        "jitnn_hip_stats": (i, [vp, i]),
        "jitnn_hip_stats_reset": (i, []),
        "jitnn_hip_block_values": (i, [i]),
        "jitnn_hip_block_bytes": (i, [i]),
        "jitnn_hip_weight_nbytes": (ll, [i, ll, ll]),
        "jitnn_hip_weight_upload": (i, [i, vp, ll, i, i, C.POINTER(vp)]),
        "jitnn_hip_weight_wrap_dev": (i, [i, vp, ll, i, i, C.POINTER(vp)]),
        "jitnn_hip_weight_free": (i, [vp]),
        "jitnn_hip_weight_info": (i, [vp, C.POINTER(i), C.POINTER(i), C.POINTER(i), C.POINTER(ll)]),
        "jitnn_hip_dequantize": (i, [vp, vp]),
        "jitnn_hip_dequantize_dev": (i, [vp, vp, vp]),
        "jitnn_hip_linear": (i, [vp, vp, i, vp, vp]),
        "jitnn_hip_linear_dev": (i, [vp, vp, i, vp, vp, vp]),
        "jitnn_hip_linear_noalloc_dev": (i, [vp, vp, i, vp, vp, vp]),
        "jitnn_hip_noalloc_scratch_bytes": (ll, []),
        "jitnn_hip_thread_release": (i, []),
        "jitnn_hip_quantize_q8_0": (i, [vp, ll, vp]),
        "jitnn_hip_quantize_q8_0_dev": (i, [vp, ll, vp, vp]),
        "jitnn_hip_probe_read_dev": (i, [vp, ll, vp]),
        "jitnn_hip_probe_read_shape_dev": (i, [vp, ll, i, i, i, vp]),
        "jitnn_hip_malloc": (i, [ll, C.POINTER(vp)]),
        "jitnn_hip_free": (i, [vp]),
        "jitnn_hip_memcpy_h2d": (i, [vp, vp, ll]),
        "jitnn_hip_memcpy_d2h": (i, [vp, vp, ll]),
        "jitnn_hip_gguf_open": (i, [C.c_char_p, C.POINTER(vp)]),
        "jitnn_hip_gguf_close": (i, [vp]),
        "jitnn_hip_gguf_header": (i, [vp, C.POINTER(i), C.POINTER(i), C.POINTER(ll), C.POINTER(ll), C.POINTER(ll)]),
        "jitnn_hip_gguf_metadata_json": (ll, [vp, C.c_char_p, ll]),
        "jitnn_hip_gguf_tensor_name": (i, [vp, ll, C.c_char_p, i]),
        "jitnn_hip_gguf_tensor_info": (i, [vp, C.c_char_p, C.POINTER(i), C.POINTER(i), C.POINTER(ll), C.POINTER(ll), C.POINTER(ll)]),
        "jitnn_hip_gguf_tensor_read": (i, [vp, C.c_char_p, vp, ll]),
        "jitnn_hip_gguf_tensor_upload": (i, [vp, C.c_char_p, C.POINTER(vp)]),
        "jitnn_hip_llama_create": (i, [i, i, i, i, i, i, i, i, C.c_float, C.c_float, C.POINTER(vp)]),
        "jitnn_hip_llama_free": (i, [vp]),
        "jitnn_hip_llama_set_weight": (i, [vp, i, i, vp]),
        "jitnn_hip_llama_set_norm": (i, [vp, i, i, vp]),
        "jitnn_hip_llama_kv_write": (i, [vp, i, i, i, vp, vp]),
        "jitnn_hip_llama_kv_read": (i, [vp, i, i, i, vp, vp]),
        "jitnn_hip_llama_decode": (i, [vp, vp, i, vp]),
        "jitnn_hip_llama_decode_dev": (i, [vp, vp, i, vp, vp]),
        "jitnn_hip_llama_prefill": (i, [vp, vp, i, i, vp]),
        "jitnn_hip_llama_set_rope_interleaved": (i, [vp, i]),
        "jitnn_hip_llama_set_embedding": (i, [vp, i, vp, ll]),
        "jitnn_hip_llama_embed_dev": (i, [vp, vp, i, vp, vp]),
        "jitnn_hip_llama_argmax_dev": (i, [vp, vp, vp, vp]),
        "jitnn_hip_llama_generate": (i, [vp, vp, i, i, i, i, vp, vp, vp]),
        "jitnn_hip_llama_prefill_dev": (i, [vp, vp, i, i, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype, fn.argtypes = res, args
    lib._signatures = sig
    return lib


lib = _bind()
_initialised = False


def last_error() -> str:
    return lib.jitnn_hip_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    """0 passes; EINVAL is the caller's misuse (ValueError, the reference's IllegalArgumentException);
    anything else is a failed native call (JitnnError)."""
    if rc == OK:
        return
    msg = f"calling {what} failed: {last_error()}"
    if rc == EINVAL:
        raise ValueError(msg)
    if rc == EIO:
        raise OSError(msg)  # the reference's IOException
    if rc == EUNSUPPORTED:
        raise UnsupportedTypeError(msg)
    raise JitnnError(msg)


def init(device: int = 0) -> None:
    global _initialised
    if not _initialised:
        check(lib.jitnn_hip_init(device), "jitnn_hip_init")
        _initialised = True


def device_info() -> dict:
    init()
    name = C.create_string_buffer(256)
    cus, hbm = C.c_int(), C.c_longlong()
    check(lib.jitnn_hip_device_info(name, 256, C.byref(cus), C.byref(hbm)), "jitnn_hip_device_info")
    return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value}


class _Stat(C.Structure):
    _fields_ = [("name", C.c_char * 32), ("calls", C.c_longlong), ("tensor_bytes", C.c_longlong)]


def stats() -> dict:
    """Calls and tensor bytes per operator since the library was loaded or stats_reset(): {name: (calls, bytes)}, bytes
    counted as the reference's telemetry counts them (jitnn-core/src/main/java/ai/beestream/jitnn/engine/Telemetry.java:222-240)."""
    n = lib.jitnn_hip_stats(None, 0)
    buf = (_Stat * n)()
    lib.jitnn_hip_stats(C.cast(buf, C.c_void_p), n)
    return {e.name.decode(): (e.calls, e.tensor_bytes) for e in buf}


def stats_reset() -> None:
    check(lib.jitnn_hip_stats_reset(), "jitnn_hip_stats_reset")
