"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, validates its
arguments without a device, and the host mirror rejects misuse before any native call."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "jitnn_hip.h").read_text()
    return sorted(set(re.findall(r"JITNN_HIP_API[^;]*?\b(jitnn_hip_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from jitnn_amd import _lib
    names = declared_symbols()
    assert len(names) >= 20
    raw = C.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/jitnn_hip.h but not exported"
    assert sorted(_lib.lib._signatures) == names, "python binding and header disagree"


def test_block_metadata_matches_reference_table():
    from jitnn_amd import DType, _lib
    table = {2: (32, 18), 3: (32, 20), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210),  # DType.java:75-98
             6: (32, 22), 7: (32, 24), 10: (256, 84), 11: (256, 110)}
    for fid, (qk, nb) in table.items():
        assert _lib.lib.jitnn_hip_block_values(fid) == qk
        assert _lib.lib.jitnn_hip_block_bytes(fid) == nb
        t = DType.from_ggml_id(fid)
        assert (t.block_values(), t.block_bytes()) == (qk, nb)
    for fid in (0, 1, 9, 15, 30, 99, -1):  # F32, F16, Q8_1, Q8_K, BF16: no block tensor type
        assert _lib.lib.jitnn_hip_block_values(fid) == 0 and _lib.lib.jitnn_hip_block_bytes(fid) == 0


def test_weight_nbytes_validation():
    from jitnn_amd import _lib
    f = _lib.lib.jitnn_hip_weight_nbytes
    assert f(12, 14336, 4096) == 33030144      # config 3
    assert f(14, 128256, 4096) == 430940160    # config 4
    assert f(8, 4096, 4096) == 17825792        # config 1
    assert f(2, 11008, 4096) == 25362432       # config 2
    assert f(12, 3, 100) == _lib.EINVAL and "multiple of its block of 256" in _lib.last_error()
    assert f(2, 3, 48) == _lib.EINVAL
    assert f(99, 3, 256) == _lib.EINVAL and "ggml type id 99" in _lib.last_error()
    assert f(12, 0, 256) == _lib.EINVAL and f(12, 3, 0) == _lib.EINVAL and f(12, -1, 256) == _lib.EINVAL
    assert f(12, 1 << 20, 1 << 20) == _lib.EINVAL  # more than 2^31-1 values


def test_null_and_size_checks_need_no_device():
    from jitnn_amd import _lib
    h = C.c_void_p()
    buf = np.zeros(144, dtype=np.uint8)
    p = buf.ctypes.data_as(C.c_void_p)
    up = _lib.lib.jitnn_hip_weight_upload
    assert up(12, None, 144, 1, 256, C.byref(h)) == _lib.EINVAL
    assert up(12, p, 143, 1, 256, C.byref(h)) == _lib.EINVAL and "needs 144 bytes, got 143" in _lib.last_error()
    assert up(12, p, 144, 1, 256, None) == _lib.EINVAL
    assert up(5, p, 144, 1, 256, C.byref(h)) == _lib.EINVAL
    assert h.value is None
    assert _lib.lib.jitnn_hip_weight_free(None) == 0
    assert _lib.lib.jitnn_hip_weight_info(None, None, None, None, None) == _lib.EINVAL
    assert _lib.lib.jitnn_hip_linear(None, p, 1, None, p) == _lib.EINVAL
    assert _lib.lib.jitnn_hip_dequantize(None, p) == _lib.EINVAL
    assert _lib.lib.jitnn_hip_quantize_q8_0(p, 33, p) == _lib.EINVAL and "multiple of 32" in _lib.last_error()
    assert _lib.lib.jitnn_hip_free(None) == 0


def test_without_a_device_calls_fail_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import jitnn_amd
    from jitnn_amd import _lib
    with pytest.raises(jitnn_amd.JitnnError, match="jitnn_hip_init failed"):
        jitnn_amd.init()
    buf = np.zeros(144, dtype=np.uint8)
    h = C.c_void_p()
    rc = _lib.lib.jitnn_hip_weight_upload(12, buf.ctypes.data_as(C.c_void_p), 144, 1, 256, C.byref(h))
    assert rc == _lib.ENODEVICE and "jitnn_hip_init" in _lib.last_error()
    with pytest.raises(jitnn_amd.JitnnError):
        jitnn_amd.Tensor.quantized(jitnn_amd.DType.Q4_K, buf, 1, 256)


def test_host_mirror_rejects_misuse_before_native_calls():
    """IllegalArgumentException cases of Tensor.persistent (Tensor.java:266-276), Gguf.linear (Gguf.java:81-83),
    Quant.quantizeQ8 (Quant.java:44-46) as ValueError."""
    from jitnn_amd import DType, Gguf, Quant, Tensor
    with pytest.raises(ValueError, match="last axis not a multiple of its block of 256"):
        Tensor.quantized(DType.Q4_K, np.zeros(144, dtype=np.uint8), 1, 100)
    with pytest.raises(ValueError, match="needs 288 array elements, got 144"):
        Tensor.quantized(DType.Q4_K, np.zeros(144, dtype=np.uint8), 2, 256)
    with pytest.raises(ValueError):
        Tensor.quantized(DType.F32, np.zeros(16, dtype=np.uint8), 4)
    with pytest.raises(ValueError, match="multiple of 32"):
        Quant.quantize_q8(Tensor.of(np.zeros((2, 33), dtype=np.float32)))
    x = Tensor.of(np.zeros((2, 8), dtype=np.float32))
    with pytest.raises(ValueError):
        Gguf.linear(x, x, None)        # FP32 "weight"
    with pytest.raises(ValueError):
        Gguf.dequantize(x)
    with pytest.raises(ValueError):
        Quant.dequantize(x)


def test_counters_list_the_operators():
    """jitnn_hip_stats needs no device: six operators, nothing counted before a call succeeds."""
    import jitnn_amd
    jitnn_amd.stats_reset()
    st = jitnn_amd.stats()
    assert list(st) == ["linear_gemv", "linear_mfma", "dequantize", "quantize_q8_0", "llama_decode", "llama_prefill"]
    assert all(v == (0, 0) for v in st.values())
