"""Shared test helpers: golden-case loader, a minimal GGUF reader, java.util.Random, error metrics.

The GGUF reader here is test infrastructure, written independently of the library's own parser so that
the two can be checked against each other.
"""
from __future__ import annotations

import struct
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
GOLDEN = ROOT / "tests" / "golden"
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

# GgufKernels format codes used by the golden manifest (GgufKernels.java:33-37) -> ggml type ids
GOLDEN_CODE_TO_GGML = {0: 2, 1: 3, 2: 12, 3: 13, 4: 14}
GGML_NAMES = {2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 10: "Q2_K", 11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K"}
HOT_FORMATS = ["Q8_0", "Q4_0", "Q4_1", "Q4_K", "Q5_K", "Q6_K"]
BLOCK = {"Q8_0": (32, 34), "Q4_0": (32, 18), "Q4_1": (32, 20), "Q5_0": (32, 22), "Q5_1": (32, 24), "Q2_K": (256, 84),
         "Q3_K": (256, 110), "Q4_K": (256, 144), "Q5_K": (256, 176), "Q6_K": (256, 210)}
GGML_ID = {v: k for k, v in GGML_NAMES.items()}


class GoldenCase:
    def __init__(self, name, op, attrs):
        self.name, self.op, self.attrs, self.arrays = name, op, attrs, {}

    def __repr__(self):
        return f"GoldenCase({self.name})"


def load_goldens() -> dict[str, GoldenCase]:
    """Same format as the reference's loader (jitnn-core/src/test/java/ai/beestream/jitnn/Golden.java:79-123)."""
    data = (GOLDEN / "golden_cases.bin").read_bytes()
    cases: dict[str, GoldenCase] = {}
    for line in (GOLDEN / "golden_cases.txt").read_text().splitlines():
        t = line.split()
        if len(t) < 2 or t[0].startswith("#"):
            continue
        if t[0] == "case":
            cases[t[1]] = GoldenCase(t[1], t[2], t[3:])
            continue
        dims = [int(d) for d in t[4:]]
        n = int(np.prod(dims)) if dims else 1
        dt = np.int32 if t[2] == "i32" else np.float32
        cases[t[0]].arrays[t[1]] = np.frombuffer(data, dtype=dt, count=n, offset=int(t[3])).reshape(dims).copy()
    return cases


class MiniGguf:
    """Just enough of GGUF v2/v3 to find tensors in the reference's fixture."""

    def __init__(self, path: Path):
        self.buf = path.read_bytes()
        self.pos = 0
        assert self.buf[:4] == b"GGUF"
        self.pos = 4
        self.version = self._u32()
        nt, nkv = self._u64(), self._u64()
        self.metadata = {}
        for _ in range(nkv):
            key = self._str()
            self.metadata[key] = self._value(self._u32())
        self.alignment = int(self.metadata.get("general.alignment", 32))
        infos = []
        for _ in range(nt):
            name = self._str()
            nd = self._u32()
            dims = [self._u64() for _ in range(nd)]
            tid = self._u32()
            off = self._u64()
            infos.append((name, dims[::-1], tid, off))
        self.data_offset = (self.pos + self.alignment - 1) // self.alignment * self.alignment
        self.tensors = {name: (shape, tid, self.data_offset + off) for name, shape, tid, off in infos}

    def _u32(self):
        v = struct.unpack_from("<I", self.buf, self.pos)[0]
        self.pos += 4
        return v

    def _u64(self):
        v = struct.unpack_from("<Q", self.buf, self.pos)[0]
        self.pos += 8
        return v

    def _str(self):
        n = self._u64()
        s = self.buf[self.pos:self.pos + n].decode("utf-8")
        self.pos += n
        return s

    def _value(self, t):
        fmts = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
        if t in fmts:
            v = struct.unpack_from(fmts[t], self.buf, self.pos)[0]
            self.pos += struct.calcsize(fmts[t])
            return v
        if t == 8:
            return self._str()
        if t == 9:
            et = self._u32()
            n = self._u64()
            return [self._value(et) for _ in range(n)]
        raise ValueError(t)

    def raw(self, name: str) -> np.ndarray:
        shape, tid, off = self.tensors[name]
        numel = int(np.prod(shape))
        if tid == 0:
            nb = numel * 4
        else:
            qk, bb = BLOCK[GGML_NAMES[tid]]
            nb = numel // qk * bb
        return np.frombuffer(self.buf, dtype=np.uint8, count=nb, offset=off).copy()

    def f32(self, name: str) -> np.ndarray:
        shape, tid, _ = self.tensors[name]
        assert tid == 0
        return self.raw(name).view(np.float32).reshape(shape)


def fixture() -> MiniGguf:
    return MiniGguf(GOLDEN / "fixture.gguf")


class JavaRandom:
    """java.util.Random (JDK-documented LCG) - used by GgufChecks to draw x (GgufChecks.java:82-90)."""

    def __init__(self, seed: int):
        self.state = (seed ^ 0x5DEECE66D) & ((1 << 48) - 1)

    def next(self, bits: int) -> int:
        self.state = (self.state * 0x5DEECE66D + 0xB) & ((1 << 48) - 1)
        return self.state >> (48 - bits)

    def next_float(self) -> np.float32:
        return np.float32(self.next(24) / float(1 << 24))


def java_string_hash(s: str) -> int:
    h = 0
    for ch in s:
        h = (31 * h + ord(ch)) & 0xFFFFFFFF
    return h - (1 << 32) if h >= (1 << 31) else h


def norm_err(actual: np.ndarray, expect: np.ndarray) -> float:
    """max|a-e| / max(|e|, 1e-6): the normalisation of GgufChecks.close (GgufChecks.java:110-120)."""
    scale = max(float(np.max(np.abs(expect))), 1e-6)
    return float(np.max(np.abs(actual.astype(np.float64) - expect.astype(np.float64)))) / scale


def checks_close(actual: np.ndarray, expect: np.ndarray, rtol: float, atol: float) -> bool:
    """|e-a| <= atol + rtol*|e| (jitnn-core/src/test/java/ai/beestream/jitnn/Checks.java:30-50)."""
    a, e = actual.astype(np.float64), expect.astype(np.float64)
    return bool(np.all(np.abs(e - a) <= atol + rtol * np.abs(e)))


def random_valid_blocks(rng: np.random.Generator, fmt: str, n: int, k: int, lo=0.002, hi=0.03) -> np.ndarray:
    """Random bytes with plausible FP16 scales, as the reference's own fixtures are made
    (scripts/gguf/gguf_fixture.py:47-52, scripts/pytorch/goldens.py:388-393)."""
    qk, nb = BLOCK[fmt]
    scale_offsets = {"Q8_0": [0], "Q4_0": [0], "Q4_1": [0, 2], "Q5_0": [0], "Q5_1": [0, 2], "Q4_K": [0, 2], "Q5_K": [0, 2],
                     "Q6_K": [208], "Q2_K": [80, 82], "Q3_K": [108]}[fmt]
    raw = rng.integers(0, 256, size=(n * k // qk, nb), dtype=np.uint8)
    for off in scale_offsets:
        raw[:, off:off + 2] = rng.uniform(lo, hi, size=(raw.shape[0], 1)).astype(np.float16).view(np.uint8)
    return raw.reshape(-1)
