"""ctypes front end of the CPU oracle (liboracle.so, built from oracle/*.c by oracle/Makefile).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg, never by the jitnn_amd package.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"

# ggml type ids (jitnn-gguf/src/main/java/ai/beestream/jitnn/gguf/GgmlType.java:27-65)
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 3, 6, 7, 8, 10, 11, 12, 13, 14
FORMATS = {"Q4_0": Q4_0, "Q4_1": Q4_1, "Q5_0": Q5_0, "Q5_1": Q5_1, "Q8_0": Q8_0, "Q2_K": Q2_K, "Q3_K": Q3_K, "Q4_K": Q4_K,
           "Q5_K": Q5_K, "Q6_K": Q6_K}

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")


def build() -> None:
    subprocess.run(["make", "-C", str(HERE), "-s"], check=True)


def _load() -> C.CDLL:
    if not LIB_PATH.exists():
        build()
    lib = C.CDLL(str(LIB_PATH))
    lib.jo_block_values.argtypes = [C.c_int]
    lib.jo_block_bytes.argtypes = [C.c_int]
    lib.jo_half_to_float.argtypes = [C.c_uint16]
    lib.jo_half_to_float.restype = C.c_float
    lib.jo_float_to_half.argtypes = [C.c_float]
    lib.jo_float_to_half.restype = C.c_uint16
    lib.jo_value.argtypes = [C.c_int, _u8p, C.c_long]
    lib.jo_value.restype = C.c_float
    lib.jo_dequantize.argtypes = [C.c_int, _u8p, C.c_long, _f32p]
    lib.jo_matvec_ref.argtypes = [C.c_int, _f32p, _u8p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.jo_linear_q8_ref.argtypes = [_f32p, _u8p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.jo_matmul_nt_ref.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.jo_matmul_nt_ref.restype = None
    lib.jo_gguf_linear.argtypes = [C.c_int, _f32p, _u8p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.jo_quantize_q8_0_ref.argtypes = [_f32p, C.c_long, _u8p]
    lib.jo_cpu_vector_lanes.argtypes = []
    lib.jo_cpu_gemm_nt.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]
    lib.jo_dequant_gemm.argtypes = [C.c_int, _f32p, _u8p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
    lib.jo_rms_norm.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_double]
    lib.jo_rms_norm.restype = None
    lib.jo_rope_tables.argtypes = [C.c_int, C.c_int, C.c_float, _f32p, _f32p]
    lib.jo_rope_tables.restype = None
    lib.jo_rope.argtypes = [_f32p, _f32p, _f32p, _f32p, C.c_long, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    lib.jo_rope.restype = None
    lib.jo_silu.argtypes = [_f32p, _f32p, C.c_long]
    lib.jo_silu.restype = None
    lib.jo_swiglu.argtypes = [_f32p, _f32p, _f32p, C.c_long]
    lib.jo_swiglu.restype = None
    lib.jo_sdpa.argtypes = [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_double]
    lib.jo_attention_decode.argtypes = [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_double]
    lib.jo_add.argtypes = [_f32p, _f32p, _f32p, C.c_long]
    lib.jo_add.restype = None
    return lib


lib = _load()


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8).reshape(-1)


def _opt(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def block_values(fmt: int) -> int:
    return lib.jo_block_values(fmt)


def block_bytes(fmt: int) -> int:
    return lib.jo_block_bytes(fmt)


def nbytes(fmt: int, numel: int) -> int:
    return numel // block_values(fmt) * block_bytes(fmt)


def dequantize(fmt: int, blocks, numel: int) -> np.ndarray:
    w = _u8(blocks)
    assert w.size == nbytes(fmt, numel), (w.size, nbytes(fmt, numel))
    y = np.empty(numel, dtype=np.float32)
    rc = lib.jo_dequantize(fmt, w, numel, y)
    assert rc == 0, rc
    return y


def matvec(fmt: int, x, blocks, n: int, k: int) -> np.ndarray:
    x = _f32(x).reshape(-1, k)
    y = np.empty((x.shape[0], n), dtype=np.float32)
    rc = lib.jo_matvec_ref(fmt, x, _u8(blocks), y, x.shape[0], n, k)
    assert rc == 0, rc
    return y


def gguf_linear(fmt: int, x, blocks, bias, n: int, k: int) -> np.ndarray:
    """Gguf.linear as the reference's host path computes it (bias may be None)."""
    x = _f32(x).reshape(-1, k)
    b = None if bias is None else _f32(bias)
    y = np.empty((x.shape[0], n), dtype=np.float32)
    rc = lib.jo_gguf_linear(fmt, x, _u8(blocks), _opt(b), y, x.shape[0], n, k)
    assert rc == 0, rc
    return y


def gguf_linear_rows_parallel(fmt: int, x, blocks, bias, n: int, k: int, threads: int = 8) -> np.ndarray:
    """gguf_linear with the output rows shared out over `threads` host threads.  Output rows are independent in the
    reference's loop, so the result is bit-identical to the one-thread call; this only shortens the wait in tests of
    whole models (the timed CPU baseline always runs the one-thread loop, which is what the reference does)."""
    from concurrent.futures import ThreadPoolExecutor

    x = _f32(x).reshape(-1, k)
    w = _u8(blocks)
    rb = nbytes(fmt, k)
    assert w.size == rb * n, (w.size, rb, n)
    b = None if bias is None else _f32(bias)
    step = max(1, (n + threads - 1) // threads)
    cuts = list(range(0, n, step))

    def part(r0):
        r1 = min(n, r0 + step)
        return gguf_linear(fmt, x, w[r0 * rb:r1 * rb], None if b is None else b[r0:r1], r1 - r0, k)

    if len(cuts) == 1:
        return part(0)
    with ThreadPoolExecutor(max_workers=threads) as pool:  # ctypes releases the GIL inside the C call
        return np.concatenate(list(pool.map(part, cuts)), axis=1)


def cpu_threads() -> int:
    """The reference's default thread count (cpu/Cpu.java:221-225): physical cores among the processors this process may
    use, at most the cores of one socket; the usable processors when the topology cannot be read."""
    import os
    try:
        usable = sorted(os.sched_getaffinity(0))
    except AttributeError:
        usable = list(range(os.cpu_count() or 1))
    cores, per_socket = set(), {}
    try:
        for c in usable:
            base = f"/sys/devices/system/cpu/cpu{c}/topology/"
            core, pkg = open(base + "core_id").read().strip(), open(base + "physical_package_id").read().strip()
            cores.add((pkg, core))
            per_socket.setdefault(pkg, set()).add(core)
    except OSError:
        return max(1, len(usable))
    return max(1, min(len(cores), max(len(v) for v in per_socket.values())))


def cpu_vector_lanes() -> int:
    return lib.jo_cpu_vector_lanes()


def dequant_gemm(fmt: int, x, blocks, bias, n: int, k: int, threads: int):
    """Gguf.linear's dequantise + FP32 GEMM branch as the reference's CPU backend runs it (oracle/jitnn_cpu_gemm.c);
    returns (y [rows, n], seconds in the one-thread dequantiser, seconds in packing + GEMM)."""
    x = _f32(x).reshape(-1, k)
    b = None if bias is None else _f32(bias)
    y = np.empty((x.shape[0], n), dtype=np.float32)
    sec = (C.c_double * 2)()
    rc = lib.jo_dequant_gemm(fmt, x, _u8(blocks), _opt(b), y, x.shape[0], n, k, threads, sec)
    assert rc == 0, rc
    return y, sec[0], sec[1]


def matmul_nt(a, b) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    c = np.empty((a.shape[0], b.shape[0]), dtype=np.float32)
    lib.jo_matmul_nt_ref(a, b, c, a.shape[0], b.shape[0], a.shape[1])
    return c


def quantize_q8_0(x) -> np.ndarray:
    x = _f32(x).reshape(-1)
    q = np.empty(x.size // 32 * 34, dtype=np.uint8)
    rc = lib.jo_quantize_q8_0_ref(x, x.size, q)
    assert rc == 0, rc
    return q


def half_to_float(h: int) -> float:
    return lib.jo_half_to_float(h)


def float_to_half(f: float) -> int:
    return lib.jo_float_to_half(f)


def rms_norm(x, w, eps: float) -> np.ndarray:
    x = _f32(x)
    cols = x.shape[-1]
    y = np.empty_like(x)
    lib.jo_rms_norm(x, _f32(w), y, x.size // cols, cols, float(np.float32(eps)))
    return y


def rope_tables(positions: int, dim: int, base: float):
    c = np.empty((positions, dim // 2), dtype=np.float32)
    s = np.empty((positions, dim // 2), dtype=np.float32)
    lib.jo_rope_tables(positions, dim, base, c, s)
    return c, s


def rope(x, base: float, offset: int, interleaved: bool, heads_axis: bool) -> np.ndarray:
    """heads_axis=False: x [..., T, D]; True: x [..., T, H, D] (Rope.apply / Rope.applyHeads)."""
    x = _f32(x)
    dim = x.shape[-1]
    seq = x.shape[-3] if heads_axis else x.shape[-2]
    group = x.shape[-2] if heads_axis else 1
    c, s = rope_tables(offset + seq, dim, base)
    out = np.empty_like(x)
    lib.jo_rope(x, out, c, s, x.size // dim, seq, dim, group, offset, int(interleaved))
    return out


def silu(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib.jo_silu(x, y, x.size)
    return y


def swiglu(gate, up) -> np.ndarray:
    gate, up = _f32(gate), _f32(up)
    y = np.empty_like(gate)
    lib.jo_swiglu(gate, up, y, gate.size)
    return y


def sdpa(q, k, v, causal: bool, scale: float | None = None) -> np.ndarray:
    """q [..., T, D], k, v [..., S, D]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    t, d = q.shape[-2:]
    s = k.shape[-2]
    z = q.size // (t * d)
    sc = float(np.float32(1.0 / np.sqrt(d))) if scale is None or scale < 0 else float(np.float32(scale))
    dv = v.shape[-1]
    o = np.empty(q.shape[:-1] + (dv,), dtype=np.float32)
    rc = lib.jo_sdpa(q, k, v, o, z, t, s, d, dv, int(causal), sc)
    assert rc == 0
    return o


def attention_decode(q, kc, vc, scale: float | None = None) -> np.ndarray:
    """q [H, D]; kc, vc [S, KV, D]."""
    q, kc, vc = _f32(q), _f32(kc), _f32(vc)
    h, d = q.shape
    s, kv, _ = kc.shape
    sc = float(np.float32(1.0 / np.sqrt(d))) if scale is None else float(np.float32(scale))
    o = np.empty_like(q)
    rc = lib.jo_attention_decode(q, kc, vc, o, h, kv, s, d, sc)
    assert rc == 0
    return o


def add(a, b) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    y = np.empty_like(a)
    lib.jo_add(a, b, y, a.size)
    return y
