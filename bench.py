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

PEAK_HBM_GBPS = 8000.0
TRAFFIC_PROFILE = ROOT / "profiles" / "gemv_q4_k_14336x4096_b1_pmc_traffic.txt"


def headline_traffic_bytes():
    """HBM bytes per launch of the headline kernel as the committed rocprofv3 --pmc summary states them (FETCH_SIZE and
    WRITE_SIZE per dispatch, each scaled by what the same counter reads for a plain copy of known size); None when the
    summary is missing or does not hold the line."""
    import re
    try:
        m = re.search(r"HBM traffic per GEMV launch =.*=\s*([0-9 ]+) bytes", TRAFFIC_PROFILE.read_text())
        return int(m.group(1).replace(" ", "")) if m else None
    except OSError:
        return None


BLOCK = {"Q8_0": (8, 32, 34), "Q4_0": (2, 32, 18), "Q4_1": (3, 32, 20), "Q4_K": (12, 256, 144), "Q5_K": (13, 256, 176),
         "Q6_K": (14, 256, 210)}


def alg_bytes(fmt: str, n: int, k: int, b: int) -> int:
    _, qk, nb = BLOCK[fmt]
    return n * k // qk * nb + b * k * 4 + b * n * 4


class Workload:
    """One GEMV configuration: `copies` device-resident copies of a quantised weight, x and y on the device."""

    def __init__(self, torch, lib, fmt: str, n: int, k: int, b: int, copies: int, seed: int):
        import quantizers  # quantizers.py beside this file: FP32 -> GGUF blocks for synthetic weights
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
        torch.cuda.synchronize()
        self.stream = torch.cuda.Stream()  # the timed launches and their events go on a stream of their own, not the legacy default stream

    def step(self, i: int, stream) -> None:
        rc = self.lib.lib.jitnn_hip_linear_dev(self.handles[i % len(self.handles)], self._xp, self.b, None, self._yp, stream)
        if rc != 0:
            self.lib.check(rc, "jitnn_hip_linear_dev")

    def time(self, steps: int, warmup: int, rotate: bool = True, events: bool = True):
        """(wall seconds, event seconds) for `steps` back-to-back launches after `warmup` untimed ones;
        rotate=False keeps to one weight copy (cache-resident figure).  events=False: no event records inside the timed
        region (a pair costs about 10 us of wall clock, half a microsecond per step of a 20-step region); the event
        seconds are then None."""
        torch = self.torch
        with torch.cuda.stream(self.stream):
            return self._time(steps, warmup, rotate, events)

    def _time(self, steps: int, warmup: int, rotate: bool, events: bool = True):
        torch = self.torch
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        m = 1 if rotate else 0
        # every weight copy gets one untimed launch first: the first kernel touch of an allocation pays for its address
        # translations, which is not what a step of a running system costs
        for i in range(len(self.handles) if rotate else 1):
            self.step(i, stream)
        for i in range(warmup):
            self.step(i * m, stream)
        # the timed loop calls the C ABI with everything bound beforehand, so that the host stays ahead of a 6-8 us kernel
        f, xp, yp, b = self.lib.lib.jitnn_hip_linear_dev, self._xp, self._yp, self.b
        order = [self.handles[(i * m) % len(self.handles)] for i in range(steps)]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        rc = 0
        t0 = time.perf_counter()
        if events:
            e0.record()
        for h in order:
            rc |= f(h, xp, b, None, yp, stream)
        if events:
            e1.record()
        # (the host polls the stream until it is done, then synchronises: a host thread parked in the blocking wait takes some
        # 10 us to wake up, half a microsecond per step of a 20-step region that is not the device's)
        cur = torch.cuda.current_stream()
        while not cur.query():
            pass
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if rc != 0:
            self.lib.check(rc, "jitnn_hip_linear_dev")
        return t1 - t0, (e0.elapsed_time(e1) * 1e-3 if events else None)

    def time_streams(self, steps: int, nstreams: int = 4):
        """GB/s of `steps` launches spread round-robin over `nstreams` streams (all of default priority), weight copies
        rotating: launches of different streams overlap, so one launch's ramp and tail run under another's rows.  A
        sustained-rate figure for callers with independent requests in flight - never the headline, which is one launch
        after the other on one stream."""
        torch = self.torch
        streams = [torch.cuda.Stream() for _ in range(nstreams)]
        ys = [torch.zeros_like(self.y) for _ in range(nstreams)]
        f = self.lib.lib.jitnn_hip_linear_dev

        def launch(i):
            s = i % nstreams
            rc = f(self.handles[i % len(self.handles)], self._xp, self.b, None, C.c_void_p(ys[s].data_ptr()), C.c_void_p(streams[s].cuda_stream))
            if rc != 0:
                self.lib.check(rc, "jitnn_hip_linear_dev")
        torch.cuda.synchronize()
        for i in range(4 * nstreams):
            launch(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            launch(i)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        same = all(bool(torch.equal(y, ys[0])) for y in ys[1:])  # (every copy holds the same weight bytes)
        return {"streams": nstreams, "steps": steps, "us_per_launch": dt / steps * 1e6, "GBps": self.bytes * steps / dt / 1e9,
                "pct_of_peak": self.bytes * steps / dt / 1e9 / PEAK_HBM_GBPS * 100, "results_equal_across_streams": same}

    def read_probe(self, steps: int, shape=None):
        """Microseconds per launch of a pure 128-bit streaming read over the same weight bytes, rotating like time();
        shape = (workgroups per CU, loads in flight per lane, non-temporal) or None for the library's default shape."""
        torch = self.torch
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        ptrs = [(C.c_void_p(t.data_ptr()), t.numel()) for t in self.weights]

        def launch(i):
            p, nb = ptrs[i % len(ptrs)]
            rc = (self.lib.lib.jitnn_hip_probe_read_dev(p, nb, stream) if shape is None
                  else self.lib.lib.jitnn_hip_probe_read_shape_dev(p, nb, shape[0], shape[1], shape[2], stream))
            if rc != 0:
                self.lib.check(rc, "jitnn_hip_probe_read")
        for i in range(len(ptrs) + 10):
            launch(i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(steps):
            launch(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    def read_probe_sweep(self, steps: int = 400):
        """The pure read over launch shapes: workgroups per CU x 16-byte loads in flight per lane x (non-)temporal loads.
        Returns the list of (shape, us) and the fastest - the ceiling a launch that only reads these bytes reaches here."""
        rows = []
        for wg in (1, 2, 4, 8, 16):
            for u in (1, 2, 4, 8, 16):
                if wg * u > 32:   # (more than 128 KiB in flight per CU: measured slower every time, not swept)
                    continue
                for nt in (0, 1):
                    rows.append({"workgroups_per_cu": wg, "loads_in_flight": u, "nontemporal": nt, "us": self.read_probe(steps, (wg, u, nt))})
        best = min(rows, key=lambda r: r["us"])
        return rows, best

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
    # the kernel's average launch duration for the roofline: a fixed, well-sampled event region whatever --steps is, behind
    # enough untimed launches for the device to have left its idle clocks (a region that starts cold reads 5 % slower)
    roof_launches = max(steps, 2000 if n < 100000 else 300)
    _, roof_ev = wl.time(roof_launches, max(warmup, roof_launches // 4))
    # The first synchronised region after the 2000-launch one pays the runtime's housekeeping for those 2000 commands (about
    # 40 us, once: 10-11 us per step over 20 steps where every later region reads 8.3): one untimed region takes it.
    wl.time(steps, warmup, events=False)
    # `value`: exactly `steps` launches between two synchronisations, nothing else in the region.  Three such regions, the median
    # reported: a region of 20 launches is 170 us of wall clock, and one host hiccup of 40 us in it reads as 25 %.
    walls = sorted(wl.time(steps, warmup, events=False)[0] for _ in range(3))
    wall = walls[1]
    _, ev = wl.time(steps, warmup)
    probe_us = wl.read_probe(400 if n < 100000 else 100)
    out = {"workload": f"{fmt} GEMV {n}x{k} batch {b}", "copies": copies, "steps": steps, "bytes_per_step": wl.bytes,
           "pure_read_us_per_launch": probe_us, "pure_read_GBps": wl.weights[0].numel() / probe_us / 1e3,
           "us_per_step_wall": wall / steps * 1e6, "us_per_step_wall_regions": [w / steps * 1e6 for w in walls], "us_per_step_events": ev / steps * 1e6, "GBps": wl.bytes * steps / wall / 1e9,
           "roofline_launches_timed": roof_launches, "us_per_launch_events": roof_ev / roof_launches * 1e6,
           "GBps_events": wl.bytes * roof_launches / roof_ev / 1e9, "pct_of_peak": wl.bytes * roof_launches / roof_ev / 1e9 / PEAK_HBM_GBPS * 100,
           "parity_norm_err": err}
    return wl, out


TILED_ROWS = 32  # jitnn.gguf.tiledRows (core/JitnnConfig.java:423-424)


def cpu_route(fmt: str, rows: int) -> str:
    """What the reference's Gguf.linear runs for this format and row count (core/ops/Gguf.java:76-98): the scalar
    FP64 loop of gguf_matvec / linear_q8_0 on one thread, or dequantise (one thread) + the multithreaded FP32 GEMM."""
    if fmt == "Q8_0":
        return "scalar"
    if (rows == 1 and fmt in ("Q4_0", "Q4_1", "Q4_K", "Q5_K", "Q6_K")) or (rows <= TILED_ROWS and fmt in ("Q4_0", "Q4_1", "Q5_K")):
        return "scalar"
    return "dequant_gemm"


def cpu_baseline(wl: Workload, budget_s: float = 12.0, max_rows: int = 32768):
    """The reference's CPU path for this workload, restated in C (oracle/), timed on this box's host cores on the same
    weight bytes and activations: Gguf.MatVec.reference / Quant.LinearQ8.reference (scalar, FP64 accumulation, ONE thread -
    what jitNN's CPU backend runs for quantised weights) where Gguf.linear takes that route, else Gguf.dequantize (one
    thread) + the packed, K-blocked, 6 x 2-vector FMA GEMM on the physical cores of one socket.  Matrices of more than
    `max_rows` weight rows are timed on their first `max_rows` rows and scaled (said in `sample`)."""
    import numpy as np
    from oracle import oracle
    fid, qk, nb = BLOCK[wl.fmt]
    n = min(wl.n, max_rows)
    rb = wl.k // qk * nb
    raw = wl.weights[0][: n * rb].cpu().numpy()
    x = wl.x.cpu().numpy()
    route = cpu_route(wl.fmt, wl.b)
    threads = 1 if route == "scalar" else oracle.cpu_threads()
    times, parts = [], []
    t_all = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        if route == "scalar":
            oracle.gguf_linear(fid, x, raw, None, n, wl.k)
        else:
            _, t_deq, t_mm = oracle.dequant_gemm(fid, x, raw, None, n, wl.k, threads)
            parts.append((t_deq, t_mm))
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all > budget_s or len(times) >= 9:
            break
    med = float(np.median(times)) * (wl.n / n)
    what = (f"the full {wl.fmt} {wl.n}x{wl.k} batch-{wl.b} linear" if n == wl.n
            else f"the first {n} of {wl.n} weight rows of the {wl.fmt} {wl.n}x{wl.k} batch-{wl.b} linear, time scaled by {wl.n / n:.3f}")
    out = {"value": wl.bytes / med / 1e9, "unit": "GB/s", "cores": threads, "kind": "port", "ms_per_step": med * 1e3, "route": route,
           "sample": f"{what}, median of {len(times)} runs of the C restatement of the reference's CPU path "
                     + ("(scalar FP64 host loop, Gguf.MatVec.reference / Quant.LinearQ8.reference, one thread)" if route == "scalar" else
                        f"(Gguf.dequantize on one thread + packed K-blocked FP32 GEMM of cpu/Gemm.java on {threads} threads, "
                        f"{oracle.cpu_vector_lanes() * 32}-bit vectors)") + ", same weight bytes and activations as the GPU"}
    if parts:
        out["dequantize_ms"] = float(np.median([p[0] for p in parts])) * (wl.n / n) * 1e3
        out["pack_and_gemm_ms"] = float(np.median([p[1] for p in parts])) * (wl.n / n) * 1e3
    return out


def host_path(torch, lib, wl: Workload, steps: int = 300):
    """The same linear through the host-pointer entry point (jitnn_hip_linear: x from host memory, y back to host memory,
    synchronous) - what a caller on the reference's Op.cpu seam gets - beside the device-resident launch."""
    import numpy as np
    x = np.ascontiguousarray(wl.x.cpu().numpy())
    y = np.empty((wl.b, wl.n), dtype=np.float32)
    xp, yp = x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p)
    f = lib.lib.jitnn_hip_linear
    for i in range(20):
        lib.check(f(wl.handles[i % len(wl.handles)], xp, wl.b, None, yp), "jitnn_hip_linear")
    t0 = time.perf_counter()
    for i in range(steps):
        f(wl.handles[i % len(wl.handles)], xp, wl.b, None, yp)
    us = (time.perf_counter() - t0) / steps * 1e6
    # the same weight copy through both entry points: the bits must agree
    lib.check(f(wl.handles[0], xp, wl.b, None, yp), "jitnn_hip_linear")
    wl.step(0, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    ok = bool(np.array_equal(y, wl.y.cpu().numpy()))
    return {"workload": f"{wl.fmt} {wl.n}x{wl.k} batch {wl.b} through jitnn_hip_linear (host pointers, synchronous, PCIe-inclusive)",
            "us_per_call": us, "GBps": wl.bytes / us / 1e3, "steps": steps, "same_bits_as_device_path": ok}


def quantized_device_weight(torch, lib, fmt, n, k, seed):
    """N(0, 0.02) weight [n, k] quantised to fmt on the device; returns the uint8 tensor."""
    import quantizers
    g = torch.Generator(device="cuda").manual_seed(seed)
    parts = []
    for r0 in range(0, n, 8192):
        w = torch.randn(min(8192, n - r0), k, generator=g, device="cuda") * 0.02
        parts.append(quantizers.quantize(fmt, w))
        del w
    return torch.cat(parts)


def wrap(lib, fmt, t, n, k):
    h = C.c_void_p()
    lib.check(lib.lib.jitnn_hip_weight_wrap_dev(BLOCK[fmt][0], C.c_void_p(t.data_ptr()), t.numel(), n, k, C.byref(h)), "wrap")
    return h


def bench_decode(torch, lib, steps, warmup):
    """BASELINE config 5: 32 layers, d_model 4096, 32/8 heads of 128, FFN 14336, vocab 128256, Q4_K_M mix (Q4_K; Q6_K for
    attn_v, ffn_down, output), FP32 KV cache pre-filled with N(0,1) at context 512, one token per step.  Every layer
    has its own copy of the weights in HBM (the values of layer 0 repeated: the step streams 4.9 GB)."""
    import jitnn_amd
    cfg = dict(layers=32, d_model=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, vocab=128256, max_ctx=520, rms_eps=1e-5, rope_theta=5e5)
    shapes = [("Q4_K", 4096, 4096), ("Q4_K", 1024, 4096), ("Q6_K", 1024, 4096), ("Q4_K", 4096, 4096), ("Q4_K", 14336, 4096),
              ("Q4_K", 14336, 4096), ("Q6_K", 4096, 14336)]
    base = [quantized_device_weight(torch, lib, f, n, k, 1050 + i) for i, (f, n, k) in enumerate(shapes)]
    dec = jitnn_amd.LlamaDecoder(**cfg)
    keep, handles = [], []
    weight_bytes = 0
    for l in range(cfg["layers"]):
        for i, (f, n, k) in enumerate(shapes):
            t = base[i] if l == 0 else base[i].clone()
            keep.append(t)
            h = wrap(lib, f, t, n, k)
            handles.append(h)
            dec.set_weight_handle(l, i, h)
            weight_bytes += t.numel()
        dec.set_norm(l, 0, torch.ones(4096).numpy())
        dec.set_norm(l, 1, torch.ones(4096).numpy())
    dec.set_norm(0, 2, torch.ones(4096).numpy())
    head = quantized_device_weight(torch, lib, "Q6_K", cfg["vocab"], 4096, 1049)
    hh = wrap(lib, "Q6_K", head, cfg["vocab"], 4096)
    dec.set_weight_handle(0, 7, hh)
    weight_bytes += head.numel()
    g = torch.Generator().manual_seed(11)
    for l in range(cfg["layers"]):
        dec.kv_write(l, 0, torch.randn(512, 8, 128, generator=g).numpy(), torch.randn(512, 8, 128, generator=g).numpy())
    x = torch.randn(4096, device="cuda")
    logits = torch.empty(cfg["vocab"], device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def run(n):
        for _ in range(n):
            dec.decode_dev(x.data_ptr(), 512, logits.data_ptr(), st)

    run(warmup)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    run(steps)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ok = bool(torch.isfinite(logits).all().item())
    kv_bytes = 32 * 2 * 513 * 8 * 128 * 4
    out = {"workload": "Llama-8B-shaped decode step, Q4_K_M mix, context 512, batch 1", "steps": steps, "ms_per_token": wall / steps * 1e3,
           "ms_per_token_events": e0.elapsed_time(e1) / steps, "tokens_per_s": steps / wall, "bytes_per_token": weight_bytes + kv_bytes,
           "GBps": (weight_bytes + kv_bytes) * steps / wall / 1e9, "pct_of_peak": (weight_bytes + kv_bytes) * steps / wall / 1e9 / PEAK_HBM_GBPS * 100,
           "launch": "direct", "logits_finite": ok}
    # the same step replayed as a HIP graph (no host launch cost per kernel)
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            dec.decode_dev(x.data_ptr(), 512, logits.data_ptr(), torch.cuda.current_stream().cuda_stream)
        ref = logits.clone()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        gw = time.perf_counter() - t0
        out["graph_ms_per_token"] = gw / steps * 1e3
        out["graph_tokens_per_s"] = steps / gw
        out["graph_matches_direct"] = bool(torch.equal(ref, logits))
    except Exception as e:  # report, never hide
        out["graph_error"] = f"{type(e).__name__}: {e}"
    # the prompt side of config 5: 512 tokens through the same 32 layers in one call (linears on the matrix-core path,
    # causal attention, keys and values appended), then the last token's logits against 512 single-token steps
    try:
        xs = torch.randn(512, 4096, device="cuda", generator=torch.Generator(device="cuda").manual_seed(12))
        pl = torch.empty(cfg["vocab"], device="cuda")
        for _ in range(2):
            dec.prefill_dev(xs.data_ptr(), 0, 512, pl.data_ptr(), st)
        torch.cuda.synchronize()
        reps = 5
        t0 = time.perf_counter()
        for _ in range(reps):
            dec.prefill_dev(xs.data_ptr(), 0, 512, pl.data_ptr(), st)
        torch.cuda.synchronize()
        pw = (time.perf_counter() - t0) / reps
        for t in range(512):
            dec.decode_dev(xs[t].data_ptr(), t, logits.data_ptr(), st)
        torch.cuda.synchronize()
        err = float((pl - logits).abs().max() / logits.abs().max())
        flops = 2.0 * 512 * sum(n * k for _, n, k in shapes) * cfg["layers"] + 2.0 * cfg["vocab"] * 4096
        out["prefill_512"] = {"workload": "the same model on a 512-token prompt from an empty cache, one call", "ms": pw * 1e3,
                              "tokens_per_s": 512 / pw, "linear_TFLOPs": flops / pw / 1e12,
                              "last_logits_vs_512_decode_steps_norm_err": err, "logits_finite": bool(torch.isfinite(pl).all().item())}
    except Exception as e:  # report, never hide
        out["prefill_512_error"] = f"{type(e).__name__}: {e}"
    # a short prompt: 40 tokens stay in the GEMV range (FP32-grade accuracy), every K-quant weight in one pass over its bytes
    try:
        xs = torch.randn(40, 4096, device="cuda", generator=torch.Generator(device="cuda").manual_seed(13))
        pl = torch.empty(cfg["vocab"], device="cuda")
        for _ in range(2):
            dec.prefill_dev(xs.data_ptr(), 0, 40, pl.data_ptr(), st)
        torch.cuda.synchronize()
        reps = 10
        t0 = time.perf_counter()
        for _ in range(reps):
            dec.prefill_dev(xs.data_ptr(), 0, 40, pl.data_ptr(), st)
        torch.cuda.synchronize()
        pw = (time.perf_counter() - t0) / reps
        for t in range(40):
            dec.decode_dev(xs[t].data_ptr(), t, logits.data_ptr(), st)
        torch.cuda.synchronize()
        err = float((pl - logits).abs().max() / logits.abs().max())
        out["prefill_40"] = {"workload": "the same model on a 40-token prompt from an empty cache, one call (GEMV range)", "ms": pw * 1e3,
                             "tokens_per_s": 40 / pw, "last_logits_vs_40_decode_steps_norm_err": err}
    except Exception as e:  # report, never hide
        out["prefill_40_error"] = f"{type(e).__name__}: {e}"
    for h in handles + [hh]:
        lib.lib.jitnn_hip_weight_free(h)
    dec.close()
    return out


def bench_prefill(torch, lib, steps=20, with_cpu=True):
    """512-token linears through the MFMA path at the layer shapes of config 5: achieved TFLOP/s (2*M*N*K per call), and beside
    each the reference's CPU route for a 512-row linear (dequantise on one thread + the multithreaded FP32 GEMM) on the same
    weight bytes and activations."""
    res = {}
    for name, fmt, n, k in (("q4_k_14336x4096", "Q4_K", 14336, 4096), ("q6_k_4096x14336", "Q6_K", 4096, 14336), ("q4_k_4096x4096", "Q4_K", 4096, 4096)):
        t = quantized_device_weight(torch, lib, fmt, n, k, 1060)
        h = wrap(lib, fmt, t, n, k)
        x = torch.randn(512, k, device="cuda")
        y = torch.empty(512, n, device="cuda")
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        call = lambda: lib.check(lib.lib.jitnn_hip_linear_dev(h, C.c_void_p(x.data_ptr()), 512, None, C.c_void_p(y.data_ptr()), st), "linear")
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        flops = 2.0 * 512 * n * k
        # parity on a sample of outputs against FP64 on the dequantised weights of a few rows
        import numpy as np
        from oracle import oracle
        sel = np.unique(np.linspace(0, n - 1, 24).astype(np.int64))
        rb = k // BLOCK[fmt][1] * BLOCK[fmt][2]
        raw = t.view(n, rb)[torch.as_tensor(sel, device="cuda")].cpu().numpy().reshape(-1)
        wd = oracle.dequantize(BLOCK[fmt][0], raw, len(sel) * k).reshape(len(sel), k).astype(np.float64)
        ref = x.cpu().numpy().astype(np.float64) @ wd.T
        err = float(np.abs(y.cpu().numpy()[:, sel] - ref).max() / np.abs(ref).max())
        res[name] = {"workload": f"{fmt} linear {n}x{k}, 512 rows (MFMA path)", "ms": ms, "TFLOPs": flops / ms / 1e9,
                     "pct_of_fp16_peak": flops / ms / 1e9 / 2500.0 * 100, "parity_norm_err": err}
        if with_cpu:
            threads = oracle.cpu_threads()
            xh, rawh = x.cpu().numpy(), t.cpu().numpy()
            runs = []
            t_all = time.perf_counter()
            while len(runs) < 3 and (not runs or time.perf_counter() - t_all < 3.0):
                t0 = time.perf_counter()
                _, t_deq, t_mm = oracle.dequant_gemm(BLOCK[fmt][0], xh, rawh, None, n, k, threads)
                runs.append((time.perf_counter() - t0, t_deq, t_mm))
            med = sorted(runs)[len(runs) // 2]
            res[name]["cpu_baseline"] = {"value": flops / med[0] / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port", "ms": med[0] * 1e3,
                                         "dequantize_ms": med[1] * 1e3, "pack_and_gemm_ms": med[2] * 1e3, "route": "dequant_gemm",
                                         "sample": f"the full {fmt} {n}x{k} linear on 512 rows, median of {len(runs)} runs of the C restatement of "
                                                   f"Gguf.dequantize (one thread) + the packed K-blocked FP32 GEMM of cpu/Gemm.java on {threads} "
                                                   f"threads, {oracle.cpu_vector_lanes() * 32}-bit vectors"}
            del xh, rawh
        lib.lib.jitnn_hip_weight_free(h)
        del t, x, y
    # the seven linears of one layer of config 5 on 512 tokens, back to back (attention and norms are not part of this path)
    layer = [("Q4_K", 4096, 4096), ("Q4_K", 1024, 4096), ("Q6_K", 1024, 4096), ("Q4_K", 4096, 4096), ("Q4_K", 14336, 4096),
             ("Q4_K", 14336, 4096), ("Q6_K", 4096, 14336)]
    ws, hs, ys = [], [], []
    for i, (fmt, n, k) in enumerate(layer):
        t = quantized_device_weight(torch, lib, fmt, n, k, 1070 + i)
        ws.append(t)
        hs.append(wrap(lib, fmt, t, n, k))
        ys.append(torch.empty(512, n, device="cuda"))
    x4, x14 = torch.randn(512, 4096, device="cuda"), torch.randn(512, 14336, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def one_layer():
        for (fmt, n, k), h, y in zip(layer, hs, ys):
            xin = x4 if k == 4096 else x14
            lib.check(lib.lib.jitnn_hip_linear_dev(h, C.c_void_p(xin.data_ptr()), 512, None, C.c_void_p(y.data_ptr()), st), "linear")

    for _ in range(3):
        one_layer()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        one_layer()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    flops = sum(2.0 * 512 * n * k for _, n, k in layer)
    res["layer_linears_512_tokens"] = {"workload": "q, k, v, o, gate, up, down of one 8B layer (Q4_K_M mix) on 512 tokens", "ms": ms,
                                       "TFLOPs": flops / ms / 1e9, "pct_of_fp16_peak": flops / ms / 1e9 / 2500.0 * 100,
                                       "tokens_per_s_32_layers_linears_only": 512.0 / (32 * ms * 1e-3)}
    for h in hs:
        lib.lib.jitnn_hip_weight_free(h)
    return res


def bench_codec(torch, lib, with_cpu):
    """The dequantiser and the Q8_0 quantiser (ops gguf_dequantize, dequantize_q8_0, quantize_q8_0) on whole weights: HIP-event
    time per call, algorithmic bytes (blocks + 4 bytes per value, read or written), bit-exactness against the oracle on the
    first rows, and the oracle's own one-thread time for the whole call (what the reference's host loop does)."""
    import numpy as np
    from oracle import oracle
    out = {}
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(fn, steps=50, warmup=5):
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / steps

    for name, fmt, n, k, seed in (("dequantize_q4_k_14336x4096", "Q4_K", 14336, 4096, 1030), ("dequantize_q6_k_4096x14336", "Q6_K", 4096, 14336, 1045),
                                  ("dequantize_q8_0_4096x4096", "Q8_0", 4096, 4096, 1010)):
        fid, qk, nb = BLOCK[fmt]
        t = quantized_device_weight(torch, lib, fmt, n, k, seed)
        h = C.c_void_p()
        lib.check(lib.lib.jitnn_hip_weight_wrap_dev(fid, C.c_void_p(t.data_ptr()), t.numel(), n, k, C.byref(h)), "wrap")
        ys = [torch.empty(n * k, dtype=torch.float32, device="cuda") for _ in range(3)]  # rotated: the Infinity Cache must not absorb the writes
        y, turn = ys[0], [0]

        def one():
            turn[0] += 1
            lib.check(lib.lib.jitnn_hip_dequantize_dev(h, C.c_void_p(ys[turn[0] % 3].data_ptr()), stream), "dequantize")
        sec = timed(one)
        nbytes = t.numel() + 4 * n * k
        rows = min(n, 64)
        raw = t[:rows * (k // qk) * nb].cpu().numpy()
        e = {"workload": f"{fmt} [{n}, {k}] blocks -> FP32, three output buffers in turn", "us": sec * 1e6, "bytes_per_call": nbytes, "GBps": nbytes / sec / 1e9,
             "pct_of_peak": nbytes / sec / 1e9 / PEAK_HBM_GBPS * 100,
             "bit_exact_first_rows": bool(np.array_equal(y[:rows * k].cpu().numpy().view(np.uint32), oracle.dequantize(fid, raw, rows * k).view(np.uint32)))}
        if with_cpu:
            sample = min(n, 2048)
            rs = t[:sample * (k // qk) * nb].cpu().numpy()
            t0 = time.perf_counter()
            oracle.dequantize(fid, rs, sample * k)
            e["cpu_baseline"] = {"ms": (time.perf_counter() - t0) * (n / sample) * 1e3, "cores": 1, "kind": "port",
                                 "sample": f"the first {sample} of {n} rows through the C restatement of the per-value decode, one thread, time scaled"}
        lib.lib.jitnn_hip_weight_free(h)
        out[name] = e
        del t, y, ys
    for name, rows, k in (("quantize_q8_0_512x14336", 512, 14336), ("quantize_q8_0_14336x4096", 14336, 4096)):
        g = torch.Generator(device="cuda").manual_seed(77)
        x = torch.randn(rows, k, generator=g, device="cuda")
        xs = [x, x.clone(), x.clone()]  # rotated inputs: three times the 235 MB of the large case
        q = torch.empty(rows * k // 32 * 34, dtype=torch.uint8, device="cuda")
        qp, turn = C.c_void_p(q.data_ptr()), [0]

        def one():
            turn[0] += 1
            lib.check(lib.lib.jitnn_hip_quantize_q8_0_dev(C.c_void_p(xs[turn[0] % 3].data_ptr()), rows * k, qp, stream), "quantize")
        sec = timed(one)
        nbytes = 4 * rows * k + q.numel()
        sample = min(rows, 64)
        e = {"workload": f"FP32 [{rows}, {k}] -> Q8_0 blocks, three input buffers in turn", "us": sec * 1e6, "bytes_per_call": nbytes, "GBps": nbytes / sec / 1e9,
             "pct_of_peak": nbytes / sec / 1e9 / PEAK_HBM_GBPS * 100,
             "bit_exact_first_rows": bool(np.array_equal(q[:sample * k // 32 * 34].cpu().numpy(), oracle.quantize_q8_0(x[:sample].cpu().numpy())))}
        if with_cpu:
            cs = min(rows, 1024)
            xs = x[:cs].cpu().numpy()
            t0 = time.perf_counter()
            oracle.quantize_q8_0(xs)
            e["cpu_baseline"] = {"ms": (time.perf_counter() - t0) * (rows / cs) * 1e3, "cores": 1, "kind": "port",
                                 "sample": f"the first {cs} of {rows} rows through the C restatement of Quant.quantize, one thread, time scaled"}
        out[name] = e
        del x, q, xs
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--quick", action="store_true", help="headline workload only (no other configs, short CPU baseline)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of extra configs to run (default all)")
    ap.add_argument("--decode", action="store_true", help="with --quick: still run the decode-step leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device-to-device copy kernel (known traffic: 256 MiB read, 256 MiB written) so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command can scale its counters")
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

    if a.calibrate_copy:
        src = torch.empty(64 << 20, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- headline: Q4_K 14336x4096 batch 1, rotating over 16 copies
    wl, head = measure(torch, lib, "Q4_K", 14336, 4096, 1, 16, a.steps, a.warmup, seed=1030)
    sweep, best = ([], None) if a.quick else wl.read_probe_sweep()
    hot_wall, hot_ev = wl.time(2000, 50, rotate=False)
    sustained = wl.time_streams(2000, 4)
    cpu = None if a.no_cpu else cpu_baseline(wl, 3.0 if a.quick else 8.0)
    host = host_path(torch, lib, wl)
    head_bytes = wl.bytes
    wl.close()

    configs = {}
    only = set(filter(None, a.only.split(",")))
    if not a.quick:
        extra = [
            ("q8_0_4096x4096_b1", "Q8_0", 4096, 4096, 1, 24, 1010),
            ("q4_0_11008x4096_b1", "Q4_0", 11008, 4096, 1, 16, 1020),
            ("q4_0_11008x4096_b4", "Q4_0", 11008, 4096, 4, 16, 1020),
            ("q4_0_11008x4096_b40", "Q4_0", 11008, 4096, 40, 16, 1020),
            ("q8_0_4096x4096_b40", "Q8_0", 4096, 4096, 40, 24, 1010),
            ("q4_k_14336x4096_b2", "Q4_K", 14336, 4096, 2, 16, 1030),
            ("q4_k_14336x4096_b8", "Q4_K", 14336, 4096, 8, 16, 1030),
            ("q4_k_14336x4096_b16", "Q4_K", 14336, 4096, 16, 16, 1030),
            ("q4_k_14336x4096_b40", "Q4_K", 14336, 4096, 40, 16, 1030),
            ("q4_k_14336x4096_b64", "Q4_K", 14336, 4096, 64, 16, 1030),
            ("q6_k_4096x14336_b40", "Q6_K", 4096, 14336, 40, 8, 1045),
            ("q6_k_128256x4096_b1", "Q6_K", 128256, 4096, 1, 2, 1040),
        ]
        for name, fmt, n, k, b, copies, seed in extra:
            if only and name not in only:
                continue
            steps = max(50, min(a.steps, 1000 if n < 100000 else 200))
            w2, out = measure(torch, lib, fmt, n, k, b, copies, steps, 20, seed)
            if not a.no_cpu:
                out["cpu_baseline"] = cpu_baseline(w2, 3.0)
            w2.close()
            configs[name] = out

    decode = prefill = codec = None
    if not a.quick or a.decode:
        if not only or "decode" in only:
            decode = bench_decode(torch, lib, steps=30, warmup=3)
        if (not only or "prefill" in only) and not a.quick:
            prefill = bench_prefill(torch, lib, with_cpu=not a.no_cpu)
        if (not only or "codec" in only) and not a.quick:
            codec = bench_codec(torch, lib, with_cpu=not a.no_cpu)

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
                   "cache_resident_GBps": head_bytes * 2000 / hot_ev / 1e9, "parity_norm_err": head["parity_norm_err"],
                   "pure_read_GBps": head["pure_read_GBps"], "pure_read_us_per_launch": head["pure_read_us_per_launch"],
                   "pure_read_best_of_sweep": best, "pure_read_sweep": sweep,
                   "gemv_over_pure_read": head["us_per_launch_events"] / (best["us"] if best else head["pure_read_us_per_launch"]),
                   "sustained_4_streams": sustained},
        "roofline": {"bound": "hbm", "achieved": head["GBps_events"], "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": head["GBps_events"] / PEAK_HBM_GBPS, "traffic": headline_traffic_bytes(),
                     "kernel": "gemv Q4_K batch 1", "us_per_launch": head["us_per_launch_events"],
                     "launches_timed": head["roofline_launches_timed"]},
        "cpu_baseline": cpu,
        "host_path": host,
        "configs": configs,
        "decode": decode,
        "prefill": prefill,
        "codec": codec,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
