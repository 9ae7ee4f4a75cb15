#!/usr/bin/env python3
"""Benchmark of the GGUF quantised-weight GEMV path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

Headline workload (BASELINE.json configs[2], batch 1): Q4_K GEMV, weight 14336x4096 drawn from N(0, 0.02)
and quantised to Q4_K, activation N(0, 1) [1, 4096].  One "step" is one GEMV launch through the C ABI
(jitnn_hip_linear_dev) with weights, activations and outputs resident in HBM.  Consecutive steps rotate over
16 distinct copies of the weight (528 MB > the 256 MB Infinity Cache) so that every step streams its weight
from HBM; the cache-resident figure (one copy) is reported separately.

Prints ONE JSON line: metric/value = achieved GB/s of algorithmic bytes (weight bytes + x + y per step) over
the wall-clock of the timed region; "roofline" prices the same bytes against the kernel's average launch
duration measured with HIP events on the launch stream; "cpu_baseline" is the CPU oracle (a C restatement of
the reference's scalar host loop, Gguf.MatVec.reference) timed on this box's host cores on the same weights
and activations; "configs" holds the other BASELINE configurations, measured the same way with fewer steps.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

PEAK_HBM_GBPS = 8000.0
BLOCK = {"Q8_0": (8, 32, 34), "Q4_0": (2, 32, 18), "Q4_1": (3, 32, 20), "Q4_K": (12, 256, 144), "Q5_K": (13, 256, 176),
         "Q6_K": (14, 256, 210)}


def alg_bytes(fmt: str, n: int, k: int, b: int) -> int:
    _, qk, nb = BLOCK[fmt]
    return n * k // qk * nb + b * k * 4 + b * n * 4


class Workload:
    """One GEMV configuration: `copies` device-resident copies of a quantised weight, x and y on the device."""

    def __init__(self, torch, lib, fmt: str, n: int, k: int, b: int, copies: int, seed: int):
        import quantizers
        self.torch, self.lib, self.fmt, self.n, self.k, self.b = torch, lib, fmt, n, k, b
        fid = BLOCK[fmt][0]
        g = torch.Generator(device="cuda").manual_seed(seed)
        blocks = []
        for r0 in range(0, n, 8192):  # quantise in row chunks: bounds the FP32 scratch for the 128256-row head
            w = torch.randn(min(8192, n - r0), k, generator=g, device="cuda") * 0.02
            if fmt == "Q8_0":  # the reference's own quantiser, through the library (Quant.java:102-118)
                q = torch.empty(w.numel() // 32 * 34, dtype=torch.uint8, device="cuda")
                lib.check(lib.lib.jitnn_hip_quantize_q8_0_dev(C.c_void_p(w.data_ptr()), w.numel(), C.c_void_p(q.data_ptr()), None), "quantize")
                torch.cuda.synchronize()
            else:
                q = quantizers.quantize(fmt, w)
            blocks.append(q)
            del w
        first = torch.cat(blocks)
        del blocks
        self.weights = [first] + [first.clone() for _ in range(copies - 1)]
        self.handles = []
        for t in self.weights:
            h = C.c_void_p()
            lib.check(lib.lib.jitnn_hip_weight_wrap_dev(fid, C.c_void_p(t.data_ptr()), t.numel(), n, k, C.byref(h)), "wrap")
            self.handles.append(h)
        gx = torch.Generator(device="cuda").manual_seed(7)
        self.x = torch.randn(b, k, generator=gx, device="cuda")
        self.y = torch.zeros(b, n, device="cuda")
        self.bytes = alg_bytes(fmt, n, k, b)
        self._xp, self._yp = C.c_void_p(self.x.data_ptr()), C.c_void_p(self.y.data_ptr())

    def step(self, i: int, stream) -> None:
        rc = self.lib.lib.jitnn_hip_linear_dev(self.handles[i % len(self.handles)], self._xp, self.b, None, self._yp, stream)
        if rc != 0:
            self.lib.check(rc, "jitnn_hip_linear_dev")

    def time(self, steps: int, warmup: int, rotate: bool = True):
        """(wall seconds, event seconds) for `steps` back-to-back launches after `warmup` untimed ones;
        rotate=False keeps to one weight copy (cache-resident figure)."""
        torch = self.torch
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        m = 1 if rotate else 0
        for i in range(warmup):
            self.step(i * m, stream)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            self.step(i * m, stream)
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return t1 - t0, e0.elapsed_time(e1) * 1e-3

    def parity(self, rows: int = 192):
        """Normalised max error of the device result against the CPU oracle on a spread of output rows."""
        import numpy as np
        from oracle import oracle
        torch = self.torch
        self.step(0, C.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        y = self.y.cpu().numpy()
        fid, qk, nb = BLOCK[self.fmt]
        rb = self.k // qk * nb
        sel = np.unique(np.linspace(0, self.n - 1, rows).astype(np.int64))
        raw = self.weights[0].view(self.n, rb)[torch.as_tensor(sel, device="cuda")].cpu().numpy().reshape(-1)
        ref = oracle.gguf_linear(fid, self.x.cpu().numpy(), raw, None, len(sel), self.k)
        scale = max(float(np.abs(ref).max()), 1e-6)
        return float(np.abs(y[:, sel].astype(np.float64) - ref).max() / scale)

    def close(self):
        for h in self.handles:
            self.lib.lib.jitnn_hip_weight_free(h)
        self.handles, self.weights = [], []
        self.torch.cuda.empty_cache()


def measure(torch, lib, fmt, n, k, b, copies, steps, warmup, seed, parity=True):
    wl = Workload(torch, lib, fmt, n, k, b, copies, seed)
    err = wl.parity() if parity else None
    wall, ev = wl.time(steps, warmup)
    out = {"workload": f"{fmt} GEMV {n}x{k} batch {b}", "copies": copies, "steps": steps, "bytes_per_step": wl.bytes,
           "us_per_step_wall": wall / steps * 1e6, "us_per_step_events": ev / steps * 1e6, "GBps": wl.bytes * steps / wall / 1e9,
           "GBps_events": wl.bytes * steps / ev / 1e9, "pct_of_peak": wl.bytes * steps / ev / 1e9 / PEAK_HBM_GBPS * 100,
           "parity_norm_err": err}
    return wl, out


def cpu_baseline(wl: Workload, budget_s: float = 12.0):
    """The oracle's restatement of Gguf.MatVec.reference (scalar, FP64 accumulation, one thread - what the reference's
    CPU backend runs for quantised weights) on the same weight bytes and activations."""
    import numpy as np
    from oracle import oracle
    fid = BLOCK[wl.fmt][0]
    raw = wl.weights[0].cpu().numpy()
    x = wl.x.cpu().numpy()
    times = []
    t_all = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        oracle.gguf_linear(fid, x, raw, None, wl.n, wl.k)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all > budget_s or len(times) >= 9:
            break
    med = float(np.median(times))
    return {"value": wl.bytes / med / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "ms_per_step": med * 1e3,
            "sample": f"the full {wl.fmt} {wl.n}x{wl.k} batch-{wl.b} GEMV, median of {len(times)} runs of the C restatement of the "
                      "reference's scalar FP64 host loop (Gguf.MatVec.reference), same weight bytes and activations as the GPU"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--quick", action="store_true", help="headline workload only (no other configs, short CPU baseline)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of extra configs to run (default all)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build measures one GPU (the path has no cross-GPU work); --gpus {a.gpus} is not supported", file=sys.stderr)
        return 2

    import torch
    from jitnn_amd import _lib as lib
    import jitnn_amd
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    jitnn_amd.init(0)
    info = jitnn_amd.device_info()

    # ---- headline: Q4_K 14336x4096 batch 1, rotating over 16 copies
    wl, head = measure(torch, lib, "Q4_K", 14336, 4096, 1, 16, a.steps, a.warmup, seed=1030)
    hot_wall, hot_ev = wl.time(min(a.steps, 2000), 50, rotate=False)
    cpu = None if a.no_cpu else cpu_baseline(wl, 3.0 if a.quick else 12.0)
    head_bytes = wl.bytes
    wl.close()

    configs = {}
    if not a.quick:
        extra = [
            ("q8_0_4096x4096_b1", "Q8_0", 4096, 4096, 1, 24, 1010),
            ("q4_0_11008x4096_b1", "Q4_0", 11008, 4096, 1, 16, 1020),
            ("q4_0_11008x4096_b4", "Q4_0", 11008, 4096, 4, 16, 1020),
            ("q4_k_14336x4096_b2", "Q4_K", 14336, 4096, 2, 16, 1030),
            ("q4_k_14336x4096_b8", "Q4_K", 14336, 4096, 8, 16, 1030),
            ("q6_k_128256x4096_b1", "Q6_K", 128256, 4096, 1, 2, 1040),
        ]
        only = set(filter(None, a.only.split(",")))
        for name, fmt, n, k, b, copies, seed in extra:
            if only and name not in only:
                continue
            steps = max(50, min(a.steps, 1000 if n < 100000 else 200))
            w2, out = measure(torch, lib, fmt, n, k, b, copies, steps, 20, seed)
            w2.close()
            configs[name] = out

    ms = head["us_per_step_wall"] / 1e3
    line = {
        "metric": "quant GEMV HBM GB/s at batch 1",
        "value": head["GBps"],
        "unit": "GB/s",
        "pct_of_peak": head["GBps"] / PEAK_HBM_GBPS * 100,
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Q4_K GEMV 14336x4096 batch 1 (BASELINE configs[2]), weights N(0,0.02) quantised to Q4_K, x N(0,1); "
                               "16 weight copies rotated per step (528 MB > 256 MB Infinity Cache)",
                   "bytes_per_step": head_bytes, "device": info["name"], "compute_units": info["compute_units"],
                   "cache_resident_GBps": head_bytes * min(a.steps, 2000) / hot_ev / 1e9, "parity_norm_err": head["parity_norm_err"]},
        "roofline": {"bound": "hbm", "achieved": head["GBps_events"], "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": head["GBps_events"] / PEAK_HBM_GBPS, "traffic": None,
                     "kernel": "gemv Q4_K batch 1", "us_per_launch": head["us_per_step_events"]},
        "cpu_baseline": cpu,
        "configs": configs,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
