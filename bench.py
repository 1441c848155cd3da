#!/usr/bin/env python3
"""Benchmark of the quantized matvec hot path on one MI355X.

A "step" is one call of the f32-in / f32-out operator (cml_matmul_f32:
activation quantize + fused dequantize-matvec) on a device-resident weight.
Inputs are synthetic: seeded N(0, 0.02) weights quantized with the host
quantizer, seeded N(0, 1) activations.  Consecutive steps rotate over enough
distinct copies of the weight that neither L2 nor the 256 MB Infinity Cache can
serve it, so the weight really streams from HBM (decode over a whole model
behaves that way); a cache-warm figure is reported beside it.

Prints one JSON line (see --help for the knobs).  The timed regions are HIP
events recorded on the stream the kernels run on; steps are replayed from a
captured graph so the GPU, not the Python launch loop, sets the pace.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from camelid_amd import binding as B  # noqa: E402
from camelid_amd.binding import DeviceBuffer, Weight, check, lib  # noqa: E402

HBM_PEAK_GBS = 8000.0    # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0  # MI355X published dense int8 matrix-core rate

# HBM bytes per launch of the dominant kernel, from hardware counters: FETCH_SIZE + WRITE_SIZE of `rocprofv3 --pmc`
# runs of this file, each scaled by what the same counter reads for `--calibrate-copy` (a plain copy of known size).
# Counters cannot be read from inside the timed run, so a line carries the reading together with where it was taken
# (`roofline.traffic_source`: the summary under profiles/ and the kernel symbol it was read for) -- a reading of another
# kernel, or none, shows as such instead of posing as this run's.  Configurations without a reading report null.
TRAFFIC_SOURCE = "profiles/hbm_traffic_fetch_write_size.txt"
TRAFFIC_READINGS: dict = {
    # config -> (bytes per launch, kernel-family counter the step must have fired for the reading to apply, kernel symbol)
    "q4k_14336x4096_n1": (33323600, "q4k.dot.wg8.fused", "gemv_q4k_cu_kernel<8, 0, 1, 8>"),                       # 1.007 x algorithmic
    "q4k_4096x14336_n1": (33677877, "q4k.dot.wg8.kcut.fused", "gemv_q4k_cu_kcut_kernel<4, 7, 0, true, 8, false>"),  # 1.017 x
    "q4k_14336x4096_n16": (34691593, "q4k.mfma.pair", "gemm_q4k_mfma_pair_kernel<false>"),                        # 1.014 x
    "q4k_14336x4096_n64": (39147913, "q4k.mfma.tile.g4t1", "gemm_q4k_mfma_kernel<4, 1, false, 1, true, false>"),  # 1.037 x
    "q6k_128256x3072_n1": (323896969, "q6k.dot.deep", "gemv_q6k_kernel<1, false, false, 4, false>"),              # 1.001 x
    "q4_0_128256x3072_n16": (252021326, "q4_0.mfma.tile", "gemm_b32_mfma_kernel<2, 1, 1, 2, 2, true, 4>"),        # 1.096 x
    "q6k_128256x3072_n16": (356232056, "q6k.mfma.tile", "gemm_q6k_mfma_kernel<1, 1, false, 2, 2, 1, true>"),      # 1.074 x
}

# rocprofv3 --kernel-trace averages of the dominant kernel, read at run time from the committed summaries (never copied
# into this file): config -> (summary under profiles/, kernel symbol prefix, launch-counter prefix the step must have fired).
ROCPROF_SUMMARIES: dict = {
    "q4k_14336x4096_n1": ("profiles/gemv_q4k_fused_quantize_14336x4096_n1.txt", "void cml::gemv_q4k_cu_kernel<8, 0, 1, 8>", "q4k.dot.wg8.fused"),
    "q4k_4096x14336_n1": ("profiles/gemv_q4k_4096x14336_n1.txt", "void cml::gemv_q4k_cu_kcut_kernel<4, 7, 0, true,", "q4k.dot.wg8.kcut.fused"),
    "q4k_14336x4096_n16": ("profiles/gemm_q4k_mfma_14336x4096_n16.txt", "void cml::gemm_q4k_mfma_pair_kernel<false>", "q4k.mfma.pair"),
    "q4k_14336x4096_n64": ("profiles/gemm_q4k_mfma_14336x4096_n64.txt", "void cml::gemm_q4k_mfma_kernel<4, 1,", "q4k.mfma.tile.g4t1"),
    "q8_0_8192x2048_n1": ("profiles/gemv_q8_0_8192x2048_n1.txt", "void cml::gemv_b32_kernel<", "q8_0.dot."),
    "q6k_128256x3072_n1": ("profiles/gemv_q6k_128256x3072_n1.txt", "void cml::gemv_q6k_kernel<", "q6k.dot."),
    "q4_0_128256x3072_n1": ("profiles/gemv_q4_0_128256x3072_n1.txt", "void cml::gemv_b32_kernel<", "q4_0.dot."),
}


def rocprof_summary(config: str, kernels_of_step) -> dict | None:
    """The profiler's average duration of this configuration's dominant kernel, from the committed summary, with its source;
    None when there is no summary, or when this run launched another kernel family than the summary was taken for."""
    entry = ROCPROF_SUMMARIES.get(config)
    if entry is None or not any(k.startswith(entry[2]) for k in kernels_of_step):
        return None
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), entry[0])
    try:
        best = None
        for line in open(path):
            if line.startswith('"' + entry[1]):
                cells = line.rsplit('",', 1)[1].split(",")   # Calls, TotalDurationNs, AverageNs, ...
                calls, avg = int(cells[0]), float(cells[2])
                if best is None or calls > best[0]:
                    best = (calls, avg, line.split('",', 1)[0].strip('"'))
        if best is None:
            return None
        return {"us_per_launch": round(best[1] / 1e3, 3), "calls": best[0], "file": entry[0], "kernel": best[2]}
    except OSError:
        return None


# name -> (format, rows, cols, tokens): BASELINE.json's configurations.
CONFIGS = {
    "q4k_14336x4096_n1": ("Q4_K", 14336, 4096, 1),   # the metric's configuration (Llama-3-8B FFN gate/up)
    "q4k_4096x14336_n1": ("Q4_K", 4096, 14336, 1),   # FFN down
    "q8_0_8192x2048_n1": ("Q8_0", 8192, 2048, 1),
    "q6k_128256x3072_n1": ("Q6_K", 128256, 3072, 1),
    "q4_0_128256x3072_n1": ("Q4_0", 128256, 3072, 1),
    "q4k_14336x4096_n2": ("Q4_K", 14336, 4096, 2),
    "q4k_14336x4096_n3": ("Q4_K", 14336, 4096, 3),
    "q4k_4096x14336_n3": ("Q4_K", 4096, 14336, 3),
    "q4k_14336x4096_n4": ("Q4_K", 14336, 4096, 4),
    "q4k_14336x4096_n8": ("Q4_K", 14336, 4096, 8),
    "q4k_14336x4096_n16": ("Q4_K", 14336, 4096, 16),
    "q4k_14336x4096_n32": ("Q4_K", 14336, 4096, 32),
    "q4k_14336x4096_n64": ("Q4_K", 14336, 4096, 64),
    "q4k_4096x14336_n16": ("Q4_K", 4096, 14336, 16),
    "q4k_4096x14336_n32": ("Q4_K", 4096, 14336, 32),
    "q4k_4096x14336_n64": ("Q4_K", 4096, 14336, 64),
    # batches on the other formats (speculative verify / prefill widths); not BASELINE configurations
    "q8_0_14336x4096_n1": ("Q8_0", 14336, 4096, 1),
    "q8_0_14336x4096_n2": ("Q8_0", 14336, 4096, 2),
    "q8_0_128256x3072_n1": ("Q8_0", 128256, 3072, 1),
    "q8_0_8192x2048_n2": ("Q8_0", 8192, 2048, 2),
    "q8_0_8192x2048_n4": ("Q8_0", 8192, 2048, 4),
    "q8_0_8192x2048_n8": ("Q8_0", 8192, 2048, 8),
    "q4_0_128256x3072_n4": ("Q4_0", 128256, 3072, 4),
    "q8_0_8192x2048_n16": ("Q8_0", 8192, 2048, 16),
    "q8_0_8192x2048_n32": ("Q8_0", 8192, 2048, 32),
    "q8_0_8192x2048_n64": ("Q8_0", 8192, 2048, 64),
    "q4_0_128256x3072_n8": ("Q4_0", 128256, 3072, 8),
    "q4_0_128256x3072_n16": ("Q4_0", 128256, 3072, 16),
    "q4_0_128256x3072_n64": ("Q4_0", 128256, 3072, 64),
    "q6k_128256x3072_n4": ("Q6_K", 128256, 3072, 4),
    "q6k_128256x3072_n8": ("Q6_K", 128256, 3072, 8),
    "q6k_128256x3072_n64": ("Q6_K", 128256, 3072, 64),
    "q6k_4096x14336_n1": ("Q6_K", 4096, 14336, 1),
    "q6k_4096x14336_n4": ("Q6_K", 4096, 14336, 4),
    "q6k_4096x14336_n8": ("Q6_K", 4096, 14336, 8),
    "q6k_4096x14336_n16": ("Q6_K", 4096, 14336, 16),
    "q6k_4096x14336_n64": ("Q6_K", 4096, 14336, 64),
    "q6k_128256x3072_n16": ("Q6_K", 128256, 3072, 16),
}


def synth_weight(fmt: int, rows: int, cols: int, seed: int) -> np.ndarray:
    L = lib()
    rb = cols // L.cml_block_values(fmt) * L.cml_block_bytes(fmt)
    out = np.empty(rows * rb, np.uint8)
    rng = np.random.default_rng(seed)
    step = max(1, (1 << 24) // cols)
    threads = min(32, os.cpu_count() or 1)
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        w = rng.standard_normal((r1 - r0, cols), dtype=np.float32) * np.float32(0.02)
        out[r0 * rb:r1 * rb] = B.quantize_weights(fmt, w, threads=threads)
    return out


class Timer:
    def __init__(self, stream):
        self.stream = stream
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        check(lib().cml_event_create(C.byref(self.e0)))
        check(lib().cml_event_create(C.byref(self.e1)))

    def start(self):
        check(lib().cml_event_record(self.e0, self.stream))

    def stop_ms(self) -> float:
        check(lib().cml_event_record(self.e1, self.stream))
        ms = C.c_float()
        check(lib().cml_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return float(ms.value)


EAGER = False   # --eager: plain stream launches in place of graph replays


class EagerSteps:
    """Stands in for a captured graph under --eager: `count` calls of fn(i) as plain stream launches."""

    def __init__(self, fn, count: int):
        self.fn, self.count = fn, count


def launch_report() -> dict:
    """{kernel-family counter: launches so far} (cml_kernel_launch_report)."""
    L = lib()
    need = int(L.cml_kernel_launch_report(None, 0))
    buf = C.create_string_buffer(need + 256)
    L.cml_kernel_launch_report(buf, len(buf))
    out = {}
    for line in buf.value.decode().splitlines():
        name, _, count = line.rpartition(" ")
        out[name] = out.get(name, 0) + int(count)
    return out


def capture(stream, fn, count: int):
    """Capture `count` calls of fn(i) on `stream` into one replayable graph."""
    if EAGER:
        return EagerSteps(fn, count)
    L = lib()
    check(L.cml_graph_begin_capture(stream), "begin capture")
    for i in range(count):
        fn(i)
    g = C.c_void_p()
    check(L.cml_graph_end_capture(stream, C.byref(g)), "end capture")
    return g


def destroy_graph(graph) -> None:
    if not isinstance(graph, EagerSteps):
        check(lib().cml_graph_destroy(graph))


def launch_graph(graph, stream) -> None:
    if isinstance(graph, EagerSteps):
        for i in range(graph.count):
            graph.fn(i)
    else:
        check(lib().cml_graph_launch(graph, stream))


def time_graph(stream, graph, timer: Timer, replays: int = 1) -> float:
    L = lib()
    check(L.cml_stream_sync(stream))
    timer.start()
    for _ in range(replays):
        launch_graph(graph, stream)
    return timer.stop_ms()


SETTLE_MS = 40.0   # GPU time replayed untimed before anything is measured (clocks ramp over a few ms)
SAMPLE_MS = 25.0   # GPU time covered by the timed replays


def time_graph_median(stream, graph, timers: list) -> tuple:
    """(median ms of one replay of `graph`, replays timed).  A graph of a few steps lasts a fraction
    of a millisecond, less than the GPU needs to reach its clocks: first the graph is replayed
    untimed for SETTLE_MS of GPU time, then replays are enqueued back to back, each between its own
    pair of events (so no host latency sits inside a timed region), and the median is reported."""
    L = lib()
    one = max(time_graph(stream, graph, timers[0]), 1e-3)
    for _ in range(min(4000, int(SETTLE_MS / one) + 1)):
        launch_graph(graph, stream)
    check(L.cml_stream_sync(stream))
    n = max(5, min(len(timers), int(SAMPLE_MS / one) + 1))
    for t in timers[:n]:
        check(L.cml_event_record(t.e0, stream))
        launch_graph(graph, stream)
        check(L.cml_event_record(t.e1, stream))
    check(L.cml_stream_sync(stream))
    ms = []
    for t in timers[:n]:
        v = C.c_float()
        check(L.cml_event_elapsed_ms(t.e0, t.e1, C.byref(v)))
        ms.append(float(v.value))
    return float(np.median(ms)), n


LAUNCH_CAL_STEPS = 64   # the constant a replay pays for being launched is measured on graphs of at most this many steps


def steps_ms(stream, fn, K: int, timers: list) -> tuple:
    """(ms per step, ms of the K-step replay, launch constant in ms, replays timed) for K calls of fn(i)
    replayed as ONE graph.  A replay pays a constant for being launched (a few microseconds: 5 % of a
    20-step graph, nothing of a 2000-step one); it is measured as 2 * T(K0) - T(2 * K0) on graphs of
    K0 = min(K, 64) and 2 * K0 steps and taken off the K-step replay.  For K <= 64 that is the
    difference of the two medians, (T(2K) - T(K)) / K; a long graph is timed as what it is, K steps in
    a row, and not by the difference of two long replays (whose second half runs a few per cent
    slower on some boxes once the chip has been kept busy for tens of milliseconds -- a difference
    of long replays reports that half alone)."""
    k0 = min(K, LAUNCH_CAL_STEPS)
    g0 = capture(stream, fn, k0)
    t0, n0 = time_graph_median(stream, g0, timers)
    g1 = capture(stream, fn, 2 * k0)
    t1, _ = time_graph_median(stream, g1, timers)
    destroy_graph(g1)
    const_ms = max(0.0, 2.0 * t0 - t1)
    if k0 == K:
        total, n = t0, n0
    else:
        gk = capture(stream, fn, K)
        total, n = time_graph_median(stream, gk, timers)
        destroy_graph(gk)
    destroy_graph(g0)
    return (total - const_ms) / K, total, const_ms, n


def cpu_topology() -> dict:
    """Logical and physical core counts and the CPU model string of this host (from /proc/cpuinfo)."""
    logical = os.cpu_count() or 1
    cores, model, family, model_no, stepping = set(), "unknown", None, None, None
    try:
        phys = core = None
        with open("/proc/cpuinfo") as f:
            for ln in f:
                key, _, val = ln.partition(":")
                key, val = key.strip(), val.strip()
                if key == "model name":
                    model = val
                elif key == "cpu family":
                    family = val
                elif key == "model":
                    model_no = val
                elif key == "stepping":
                    stepping = val
                elif key == "physical id":
                    phys = val
                elif key == "core id":
                    core = val
                elif not key and phys is not None:
                    cores.add((phys, core))
                    phys = core = None
            if phys is not None:
                cores.add((phys, core))
    except OSError:
        pass
    hyper = ""
    try:
        with open("/proc/cpuinfo") as f:
            if " hypervisor" in f.read():
                hyper = ", virtual machine"
    except OSError:
        pass
    if family is not None:
        model = f"{model} (family {family} model {model_no} stepping {stepping}{hyper})"
    return {"cores_logical": logical, "cores_physical": len(cores) or logical, "cpu_model": model}


def _time_cpu(call, budget_s: float, min_calls: int = 2, max_calls: int = 200) -> list:
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_calls or (time.perf_counter() < t_end and len(times) < max_calls):
        t0 = time.perf_counter()
        call()
        times.append(time.perf_counter() - t0)
    return times


def cpu_baseline(fmt: int, wire: np.ndarray, rows: int, cols: int, x: np.ndarray, alg_bytes: int, budget_s: float):
    """The CPU path, restated (oracle/): same weight, same activation, on the host cores: one
    thread, one thread per physical core, and the best of a sweep over thread counts."""
    import oracle  # test infrastructure; used here only as the timed CPU baseline
    topo = cpu_topology()
    logical, physical = topo["cores_logical"], topo["cores_physical"]
    order = oracle.ORDER_PRIMARY

    def run(threads):
        return lambda: oracle.matmul(fmt, wire, cols, x, order=order, threads=threads)

    counts = sorted({1, physical, logical} | {c for c in (2, 4, 8, 16, 32, 64, 128) if c <= logical})
    run(min(physical, 16))()  # warm-up: pages in the weight
    share = budget_s / (len(counts) + 2)
    sweep = {c: float(np.median(_time_cpu(run(c), share if c > 1 else min(share, 1.5), min_calls=2))) for c in counts}
    best = min(sweep, key=sweep.get)
    times = _time_cpu(run(best), 2 * share, min_calls=3)  # the reported figure: a longer run at the best count
    med = float(np.median(times))
    return {
        "value": round(alg_bytes / med / 1e9, 3), "unit": "GB/s", "cores": best, "kind": "port",
        "us_per_call": round(med * 1e6, 1), "best_threads": best, **topo,
        "us_per_call_1_thread": round(sweep[1] * 1e6, 1),
        "us_per_call_physical_cores": round(sweep[physical] * 1e6, 1),
        "us_per_call_by_threads": {str(c): round(t * 1e6, 1) for c, t in sweep.items()},
        "sample": f"{len(times)} full calls of the same {rows}x{cols} matvec (quantize + row dots) at {best} threads, median; "
                  f"thread sweep {counts} with a few calls each",
    }


MOE_CONFIGS = {
    # name -> (variant, format, experts, top_k, hidden, ff, tokens)
    # Mixtral-8x7B-shaped expert FFN in Q4_K: separate gate / up tensors, top-k softmax routing, silu
    "moe_q4k_8x14336x4096_t1": ("mixtral", "Q4_K", 8, 2, 4096, 14336, 1),
    "moe_q4k_8x14336x4096_t32": ("mixtral", "Q4_K", 8, 2, 4096, 14336, 32),
    "moe_q4k_8x14336x4096_t64": ("mixtral", "Q4_K", 8, 2, 4096, 14336, 64),   # short prefill: 16 assignments per expert on average
    "moe_q4k_8x14336x4096_t128": ("mixtral", "Q4_K", 8, 2, 4096, 14336, 128),
    # Mixtral-8x22B-shaped: hidden 6144 (rows of 24 super-blocks), ff 16384
    "moe_q4k_8x16384x6144_t1": ("mixtral", "Q4_K", 8, 2, 6144, 16384, 1),
    "moe_q4k_8x16384x6144_t32": ("mixtral", "Q4_K", 8, 2, 6144, 16384, 32),
    # Gemma-4 26B-shaped expert lane in Q4_0: fused gate|up tensor, full-softmax routing with
    # per-expert down scales, gelu_tanh
    "moe_q4_0_128x704x2816_t1": ("gemma4", "Q4_0", 128, 8, 2816, 704, 1),
    "moe_q4_0_128x704x2816_t32": ("gemma4", "Q4_0", 128, 8, 2816, 704, 32),
}


def bench_moe(name: str, K: int, W: int, seed: int, cpu_seconds: float) -> int:
    """One step = route + the whole expert FFN (gate and up projections, activation * up ->
    quantize, down projection, weighted sum) for all tokens, on stacked expert tensors resident
    in HBM.  Steps rotate over several routing inputs and several copies of the layer, so different
    experts are touched and nothing is served from cache."""
    L = lib()
    variant, fmt_name, E, k, hidden, ff, T = MOE_CONFIGS[name]
    gemma = variant == "gemma4"
    fmt = B.FORMATS[fmt_name]
    # values do not matter for timing: one expert's worth of seeded weights, repeated for every expert
    g1 = synth_weight(fmt, ff, hidden, seed)
    u1 = synth_weight(fmt, ff, hidden, seed + 1)
    d1 = synth_weight(fmt, hidden, ff, seed + 2)
    expert_bytes = g1.nbytes + u1.nbytes + d1.nbytes
    down_w = np.tile(d1, E)
    n_layers = max(2, min(16, -(-600_000_000 // (E * expert_bytes))))
    if gemma:
        gate_w, up_w = np.tile(np.concatenate([g1, u1]), E), None
        layers = [(Weight.upload(fmt, E * 2 * ff, hidden, gate_w), None, Weight.upload(fmt, E * hidden, ff, down_w))
                  for _ in range(n_layers)]
    else:
        gate_w, up_w = np.tile(g1, E), np.tile(u1, E)
        layers = [(Weight.upload(fmt, E * ff, hidden, gate_w), Weight.upload(fmt, E * ff, hidden, up_w),
                   Weight.upload(fmt, E * hidden, ff, down_w)) for _ in range(n_layers)]
    rng = np.random.default_rng(seed + 3)
    n_sets = 8
    logits = rng.standard_normal((n_sets, T, E)).astype(np.float32)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    down_scale = rng.uniform(0.5, 2.0, E).astype(np.float32)
    touched = [len(set(np.argsort(-logits[s], axis=1, kind="stable")[:, :k].reshape(-1))) for s in range(n_sets)]
    alg_bytes = float(np.mean(touched)) * expert_bytes + 2 * 4 * T * hidden + 4 * T * E

    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    ld = [DeviceBuffer.from_numpy(logits[s]) for s in range(n_sets)]
    xd = DeviceBuffer.from_numpy(x)
    dsd = DeviceBuffer.from_numpy(down_scale)
    idx = DeviceBuffer(T * k * 4)
    wts = DeviceBuffer(T * k * 4)
    out = DeviceBuffer(T * hidden * 4)
    ws_bytes = L.cml_moe_workspace_bytes(fmt, hidden, ff, T, k, E)
    ws = DeviceBuffer(ws_bytes)
    timer = Timer(stream)

    # CAMELID_BENCH_MOE_TWO_CALLS=1: the Mixtral-shaped step as cml_moe_route_top_k + cml_moe_ffn (the routing always a launch of its own)
    two_calls = os.environ.get("CAMELID_BENCH_MOE_TWO_CALLS", "0") == "1"

    def step(i):
        gate, up, down = layers[i % n_layers]
        if gemma:
            check(L.cml_moe_route_softmax_top_k(ld[i % n_sets].ptr, T, E, k, dsd.ptr, idx.ptr, wts.ptr, stream),
                  "cml_moe_route_softmax_top_k")
            check(L.cml_moe_ffn_ex(gate.handle, None, down.handle, E, k, idx.ptr, wts.ptr, xd.ptr, T, out.ptr,
                                   ws.ptr, ws_bytes, 1, stream), "cml_moe_ffn_ex")
        elif two_calls:
            check(L.cml_moe_route_top_k(ld[i % n_sets].ptr, T, E, k, idx.ptr, wts.ptr, stream), "cml_moe_route_top_k")
            check(L.cml_moe_ffn(gate.handle, up.handle, down.handle, E, k, idx.ptr, wts.ptr, xd.ptr, T, out.ptr,
                                ws.ptr, ws_bytes, stream), "cml_moe_ffn")
        else:
            # router logits in: routing and expert lane as one call (one token: routed inside the gate|up launch)
            check(L.cml_moe_ffn_logits(gate.handle, up.handle, down.handle, E, k, ld[i % n_sets].ptr, xd.ptr, T, out.ptr,
                                       ws.ptr, ws_bytes, stream), "cml_moe_ffn_logits")

    for i in range(W):
        step(i)
    check(L.cml_stream_sync(stream))
    timers = [timer] + [Timer(stream) for _ in range(31)]
    ms = steps_ms(stream, step, K, timers)[0]
    check(L.cml_stream_sync(stream))
    if not np.all(np.isfinite(out.to_numpy(np.float32, (T, hidden)))):
        print("non-finite output", file=sys.stderr)
        return 4
    gbs = alg_bytes / (ms * 1e-3) / 1e9
    if gemma:
        # one token: route, gate|up (quantizes the token itself), down (gelu*up->Q8_0 in its prologue), weighted sum;
        # more: route, plan, quantize, gate|up, gelu*up->Q8_0, down, weighted sum
        launches, kernel = (4 if T == 1 else 7), "gemv_b32_grouped_kernel (2 launches of the step)"
        what = "route (full softmax) + fused gate|up matvec + gelu_tanh*up->Q8_0 + down matvec + weighted sum, graph replay"
    else:
        # one token: gate and up in one launch (routes and quantizes the token itself), silu*up->Q8_K, down + weighted sum in one launch;
        # more: route, plan, quantize, gate and up in one launch, silu*up->Q8_K, down, weighted sum
        routed_in_launch = T == 1 and not two_calls and not (os.environ.get("CAMELID_HIP_TUNING", "0") not in ("", "0") and os.environ.get("CAMELID_HIP_MOE_FOLD_ROUTE", "1") == "0")
        launches, kernel = ((3 if routed_in_launch else 4) if T == 1 else 7), "gemv_q4k_kernel / gemm_q4k_mfma_kernel grouped by expert (2-3 launches of the step)"
        what = ("route + gate/up matvecs + silu*up->Q8_K + down matvec + weighted sum (cml_moe_ffn_logits; one token: the routing inside "
                "the gate|up launch, the weighted sum inside the down launch), graph replay")
    line = {
        "metric": f"{fmt_name} mixture-of-experts FFN µs + achieved HBM GB/s, {E} experts top-{k}, {ff}x{hidden}, {T} token(s)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms, 6), "us_per_call": round(ms * 1e3, 3),
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": name, "variant": variant, "format": fmt_name, "experts": E, "top_k": k, "hidden": hidden, "ff": ff,
                   "tokens": T, "algorithmic_bytes_per_call": int(alg_bytes), "mean_experts_touched": float(np.mean(touched)),
                   "layer_copies": n_layers, "step": what, "launches_per_step": launches},
        # the expert matvec launches carry the bytes; the figure is for the whole step
        "roofline": {"bound": "hbm", "kernel": kernel,
                     "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "us_per_launch": round(ms * 1e3, 3), "note": "whole step, all launches"},
    }
    if cpu_seconds > 0:
        import oracle  # test infrastructure; used here only as the timed CPU baseline
        threads = cpu_topology()["cores_physical"]
        times = []
        t_end = time.perf_counter() + cpu_seconds
        while len(times) < 2 or (time.perf_counter() < t_end and len(times) < 50):
            t0 = time.perf_counter()
            oracle.moe_ffn_ex(fmt, gate_w, up_w, down_w, E, k, hidden, ff, logits[len(times) % n_sets], x,
                              variant=1 if gemma else 0, down_scale=down_scale if gemma else None, threads=threads)
            times.append(time.perf_counter() - t0)
        med = float(np.median(times))
        line["cpu_baseline"] = {"value": round(alg_bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
                                "us_per_call": round(med * 1e6, 1),
                                "sample": f"{len(times)} full calls of the same expert FFN ({T} token(s)), median"}
    print(json.dumps(line, ensure_ascii=False))
    return 0


PAIR_CONFIGS = {
    # name -> (format, rows, cols): one token against TWO weights of one shape that read it (gate and up of a dense FFN)
    "q4k_pair_14336x4096": ("Q4_K", 14336, 4096),
    "q4k_pair_4096x4096": ("Q4_K", 4096, 4096),
    "q8_0_pair_8192x2048": ("Q8_0", 8192, 2048),
    "q4_0_pair_14336x4096": ("Q4_0", 14336, 4096),
}


def bench_pair(name: str, K: int, W: int, seed: int) -> int:
    """cml_matmul_f32_pair: one f32 token, two weights, one launch where the shape is served; beside it
    the same step as two cml_matmul_f32 calls."""
    L = lib()
    fmt_name, rows, cols = PAIR_CONFIGS[name]
    fmt = B.FORMATS[fmt_name]
    wire_a, wire_b = synth_weight(fmt, rows, cols, seed), synth_weight(fmt, rows, cols, seed + 7)
    copies = max(2, min(32, -(-600_000_000 // (2 * wire_a.nbytes))))
    wa = [Weight.upload(fmt, rows, cols, wire_a) for _ in range(copies)]
    wb = [Weight.upload(fmt, rows, cols, wire_b) for _ in range(copies)]
    x = np.random.default_rng(seed + 1).standard_normal((1, cols)).astype(np.float32)
    alg = 2 * wire_a.nbytes + 4 * cols + 2 * 4 * rows
    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    xd = DeviceBuffer.from_numpy(x)
    ws_bytes = L.cml_matmul_workspace_bytes(fmt, cols, 1)
    ws = DeviceBuffer(ws_bytes)
    oa, ob = DeviceBuffer(rows * 4), DeviceBuffer(rows * 4)

    def pair(i):
        check(L.cml_matmul_f32_pair(wa[i % copies].handle, wb[i % copies].handle, xd.ptr, oa.ptr, ob.ptr, ws.ptr, ws_bytes, stream),
              "cml_matmul_f32_pair")

    def two(i):
        check(L.cml_matmul_f32(wa[i % copies].handle, xd.ptr, 1, oa.ptr, ws.ptr, ws_bytes, stream), "cml_matmul_f32")
        check(L.cml_matmul_f32(wb[i % copies].handle, xd.ptr, 1, ob.ptr, ws.ptr, ws_bytes, stream), "cml_matmul_f32")

    for i in range(W):
        pair(i)
    check(L.cml_stream_sync(stream))
    timers = [Timer(stream) for _ in range(32)]
    ms = steps_ms(stream, pair, K, timers)[0]
    ms_two = steps_ms(stream, two, K, timers)[0]
    check(L.cml_stream_sync(stream))
    got = oa.to_numpy(np.float32, (rows,))
    if not np.all(np.isfinite(got)):
        print("non-finite output", file=sys.stderr)
        return 4
    gbs = alg / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": f"{fmt_name} matvec pair (one token, two weights) µs + achieved HBM GB/s, 2 x {rows}x{cols}",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms, 6),
        "us_per_call": round(ms * 1e3, 3), "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": name, "format": fmt_name, "rows": rows, "cols": cols, "tokens": 1, "weights": 2,
                   "algorithmic_bytes_per_call": alg, "weight_copies_rotated": copies,
                   "step": "cml_matmul_f32_pair: quantize the token + both fused dequantize-matvecs, graph replay",
                   "as_two_calls_us": round(ms_two * 1e3, 3)},
        "roofline": {"bound": "hbm", "kernel": "the single-token matvec kernel of the format, grid.z = 2 (one launch)", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "us_per_launch": round(ms * 1e3, 3)}}, ensure_ascii=False))
    return 0


MULTI_CONFIGS = {
    # name -> (format, [rows of each weight], cols): one token against several weights that read it
    "q4k_qkv_4096": ("Q4_K", [4096, 1024, 1024], 4096),           # q | k | v of a Llama-3-8B attention block (grouped-query: 8 KV heads)
    "q4k_qkv_gate_up_4096": ("Q4_K", [14336, 14336], 4096),       # gate | up through the same entry
    "q4k_qkv_3584": ("Q4_K", [3584, 512, 512], 3584),             # Qwen2.5-7B-shaped q | k | v
    "q8_0_qkv_4096": ("Q8_0", [4096, 1024, 1024], 4096),          # the same attention block in the 32-value block formats
    "q4_0_qkv_4096": ("Q4_0", [4096, 1024, 1024], 4096),
    "q6k_qkv_4096": ("Q6_K", [4096, 1024, 1024], 4096),
}


def bench_multi(name: str, K: int, W: int, seed: int) -> int:
    """cml_matmul_f32_multi: one f32 token, several weights, one launch where the set is served; beside it the
    same step as one cml_matmul_f32 call per weight."""
    L = lib()
    fmt_name, rows_list, cols = MULTI_CONFIGS[name]
    fmt = B.FORMATS[fmt_name]
    n = len(rows_list)
    wires = [synth_weight(fmt, r, cols, seed + 11 * j) for j, r in enumerate(rows_list)]
    total = sum(w.nbytes for w in wires)
    copies = max(2, min(32, -(-600_000_000 // total)))
    sets = [[Weight.upload(fmt, r, cols, wires[j]) for j, r in enumerate(rows_list)] for _ in range(copies)]
    x = np.random.default_rng(seed + 1).standard_normal((1, cols)).astype(np.float32)
    alg = total + 4 * cols + 4 * sum(rows_list)
    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    xd = DeviceBuffer.from_numpy(x)
    ws_bytes = L.cml_matmul_workspace_bytes(fmt, cols, 1)
    ws = DeviceBuffer(ws_bytes)
    outs = [DeviceBuffer(r * 4) for r in rows_list]
    optrs = (C.c_void_p * n)(*[o.ptr for o in outs])
    handles = [(C.c_void_p * n)(*[w.handle for w in st]) for st in sets]

    def multi(i):
        check(L.cml_matmul_f32_multi(handles[i % copies], n, xd.ptr, optrs, ws.ptr, ws_bytes, stream), "cml_matmul_f32_multi")

    def singles(i):
        for j, w in enumerate(sets[i % copies]):
            check(L.cml_matmul_f32(w.handle, xd.ptr, 1, outs[j].ptr, ws.ptr, ws_bytes, stream), "cml_matmul_f32")

    for i in range(W):
        multi(i)
    check(L.cml_stream_sync(stream))
    timers = [Timer(stream) for _ in range(32)]
    before = L.cml_kernel_launches(b"")
    multi(0)
    launches = L.cml_kernel_launches(b"") - before
    ms = steps_ms(stream, multi, K, timers)[0]
    ms_single = steps_ms(stream, singles, K, timers)[0]
    check(L.cml_stream_sync(stream))
    if not all(np.all(np.isfinite(o.to_numpy(np.float32, (r,)))) for o, r in zip(outs, rows_list)):
        print("non-finite output", file=sys.stderr)
        return 4
    gbs = alg / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": f"{fmt_name} matvec of {n} weights off one token µs + achieved HBM GB/s, rows {rows_list} x {cols}",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms, 6),
        "us_per_call": round(ms * 1e3, 3), "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": name, "format": fmt_name, "rows": rows_list, "cols": cols, "tokens": 1, "weights": n,
                   "algorithmic_bytes_per_call": alg, "weight_copies_rotated": copies, "launches_per_step": int(launches),
                   "step": "cml_matmul_f32_multi: quantize the token + every fused dequantize-matvec, graph replay",
                   "as_single_calls_us": round(ms_single * 1e3, 3)},
        "roofline": {"bound": "hbm", "kernel": "the single-token Q4_K matvec kernel, the weights' workgroups end to end in one launch",
                     "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "us_per_launch": round(ms * 1e3, 3)}}, ensure_ascii=False))
    return 0


PRODUCER_CONFIGS = {
    # name -> (cols, tokens): rms_norm fused with the Q8_K quantizer, the step upstream of a projection
    "rmsnorm_q8k_4096_t1": (4096, 1),
    "rmsnorm_q8k_4096_t32": (4096, 32),
}


def bench_producer(name: str, K: int, W: int, seed: int) -> int:
    """rms_norm + Q8_K quantize of `tokens` rows.  Latency-bound by construction: the reference's
    left-to-right sum of squares runs in one lane per row."""
    L = lib()
    cols, T = PRODUCER_CONFIGS[name]
    rng = np.random.default_rng(seed)
    xd = DeviceBuffer.from_numpy(rng.standard_normal((T, cols)).astype(np.float32))
    wd = DeviceBuffer.from_numpy((rng.standard_normal(cols) * 0.5 + 1).astype(np.float32))
    qd, sd = DeviceBuffer(T * cols), DeviceBuffer(T * (cols // 256) * 4)
    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    timer = Timer(stream)

    def step(i):
        check(L.cml_rms_norm_quantize(2, xd.ptr, wd.ptr, 1e-6, T, cols, None, qd.ptr, sd.ptr, stream), "cml_rms_norm_quantize")

    for i in range(W):
        step(i)
    ms = steps_ms(stream, step, K, [timer] + [Timer(stream) for _ in range(31)])[0]
    alg = T * cols * 5 + cols * 4 + T * (cols // 256) * 4
    print(json.dumps({"metric": f"rms_norm + Q8_K quantize µs, {cols} values x {T} token(s)", "value": round(ms * 1e3, 3), "unit": "us",
                      "higher_is_better": False, "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms, 6),
                      "dtype": "f32", "data": "synthetic", "config": {"workload": name, "algorithmic_bytes_per_call": alg},
                      "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 6), "traffic": None,
                                   "note": "latency-bound: one lane sums the squares in the reference's order"}}, ensure_ascii=False))
    return 0


def time_read_only(stream, timers, nbytes: int, K: int, in_flight: int, groups: int, bufs=None):
    """us per launch of the read-only yardstick over buffers rotated like the weights."""
    L = lib()
    if bufs is None:
        n = max(2, min(32, -(-600_000_000 // nbytes)))
        bufs = [DeviceBuffer(nbytes) for _ in range(n)]
        for b in bufs:
            b.fill(0x5a)

    def step(i):
        check(L.cml_calibrate_read(bufs[i % len(bufs)].ptr, nbytes, in_flight, groups, stream), "cml_calibrate_read")

    for i in range(8):
        step(i)
    ms = steps_ms(stream, step, K, timers)[0]
    return ms * 1e3, bufs


def calibrate_read(nbytes: int, K: int, W: int) -> int:
    """Read-only launches of `nbytes` over rotating buffers, at several depths and grid sizes."""
    L = lib()
    nbytes = max(16, nbytes // 16 * 16)
    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    timers = [Timer(stream) for _ in range(32)]
    rows, bufs, best = [], None, None
    for groups in (256, 512, 1024, 2048, 4096, 8192):
        for in_flight in (2, 4, 8):
            us, bufs = time_read_only(stream, timers, nbytes, K, in_flight, groups, bufs)
            rows.append({"workgroups": groups, "loads_in_flight_per_lane": in_flight, "us_per_launch": round(us, 3),
                         "gbs": round(nbytes / us / 1e3, 1)})
            if best is None or us < best["us_per_launch"]:
                best = rows[-1]
    print(json.dumps({"metric": "read-only launch (non-temporal 16-byte loads, grid-stride)", "value": best["gbs"], "unit": "GB/s",
                      "bytes_read": nbytes, "us_per_launch": best["us_per_launch"], "best": best,
                      "frac_of_hbm_peak": round(best["gbs"] / HBM_PEAK_GBS, 4), "steps": K, "warmup": W, "n_gpus": 1, "sweep": rows}))
    return 0


def calibrate_copy(nbytes: int, K: int, W: int) -> int:
    """Plain copy kernel over rotating buffers: what this box's HBM gives a kernel with no arithmetic."""
    L = lib()
    nbytes = max(16, nbytes // 16 * 16)
    pairs = max(2, min(16, -(-600_000_000 // (2 * nbytes))))
    src = [DeviceBuffer(nbytes) for _ in range(pairs)]
    dst = [DeviceBuffer(nbytes) for _ in range(pairs)]
    for b in src:
        b.fill(1)
    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    timer = Timer(stream)

    def step(i):
        check(L.cml_copy_dev(dst[i % pairs].ptr, src[i % pairs].ptr, nbytes, stream), "cml_copy_dev")

    for i in range(W):
        step(i)
    ms = steps_ms(stream, step, K, [timer] + [Timer(stream) for _ in range(31)])[0]
    check(L.cml_stream_sync(stream))
    gbs = 2 * nbytes / (ms * 1e-3) / 1e9
    print(json.dumps({"metric": "plain device copy (read + write)", "value": round(gbs, 2), "unit": "GB/s",
                      "bytes_copied": nbytes, "bytes_moved": 2 * nbytes, "us_per_launch": round(ms * 1e3, 3),
                      "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "steps": K, "warmup": W, "n_gpus": 1}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", default="q4k_14336x4096_n1",
                    help="one of: " + ", ".join(sorted(CONFIGS) + sorted(MOE_CONFIGS) + sorted(PAIR_CONFIGS) + sorted(MULTI_CONFIGS) + sorted(PRODUCER_CONFIGS))
                    + "; or any <format>_<rows>x<cols>_n<tokens>, <format>_pair_<rows>x<cols>, <format>_multi_<rows>+<rows>[+...]x<cols>, "
                      "e.g. q8_0_14336x4352_n1, q4k_pair_11008x4096, q4k_multi_4096+1024+1024x4096")
    ap.add_argument("--copies", type=int, default=0, help="distinct weight copies to rotate over (0 = enough for ~600 MB)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="time budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--eager", action="store_true",
                    help="plain stream launches in place of graph replays: for profilers that cannot follow a graph launch "
                         "(kernel durations are the same; per-step times then include the host's launch cost)")
    ap.add_argument("--cold-only", action="store_true",
                    help="skip the cache-warm leg and the eager loop (every launch of the dominant kernel is then "
                         "cache-cold, so a profiler's average duration is comparable with roofline.us_per_launch)")
    ap.add_argument("--calibrate-read", type=int, default=0, metavar="BYTES",
                    help="instead of a matvec, time a launch that only reads BYTES (grid-stride non-temporal loads, "
                         "several depths and grid sizes): what a read-only launch of that size reaches on this chip")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="BYTES",
                    help="instead of a matvec, time a plain device copy of BYTES (the yardstick for byte counters)")
    args = ap.parse_args()
    global EAGER
    EAGER = args.eager
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no collectives and every box here has one GPU; "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    L = lib()
    if L.cml_available() != 1:
        print("no usable gfx950 device: " + L.cml_last_error().decode(), file=sys.stderr)
        return 3
    B.init(0)
    if args.calibrate_read:
        return calibrate_read(args.calibrate_read, max(1, args.steps), max(0, args.warmup))
    if args.calibrate_copy:
        return calibrate_copy(args.calibrate_copy, max(1, args.steps), max(0, args.warmup))
    if args.config in PRODUCER_CONFIGS:
        return bench_producer(args.config, max(1, args.steps), max(0, args.warmup), args.seed)
    fmt_names = {"q8_0": "Q8_0", "q4_0": "Q4_0", "q4k": "Q4_K", "q6k": "Q6_K"}
    m = re.fullmatch(r"(q8_0|q4_0|q4k|q6k)_pair_(\d+)x(\d+)", args.config)
    if m and args.config not in PAIR_CONFIGS:
        PAIR_CONFIGS[args.config] = (fmt_names[m.group(1)], int(m.group(2)), int(m.group(3)))
    m = re.fullmatch(r"(q8_0|q4_0|q4k|q6k)_multi_(\d+(?:\+\d+){1,3})x(\d+)", args.config)
    if m:
        MULTI_CONFIGS[args.config] = (fmt_names[m.group(1)], [int(r) for r in m.group(2).split("+")], int(m.group(3)))
    if args.config in PAIR_CONFIGS:
        return bench_pair(args.config, max(1, args.steps), max(0, args.warmup), args.seed)
    if args.config in MULTI_CONFIGS:
        return bench_multi(args.config, max(1, args.steps), max(0, args.warmup), args.seed)
    if args.config in MOE_CONFIGS:
        return bench_moe(args.config, max(1, args.steps), max(0, args.warmup), args.seed, args.cpu_seconds)
    if args.config in CONFIGS:
        fmt_name, rows, cols, n = CONFIGS[args.config]
    else:
        m = re.fullmatch(r"(q8_0|q4_0|q4k|q6k)_(\d+)x(\d+)_n(\d+)", args.config)
        if not m:
            print(f"unknown --config {args.config}", file=sys.stderr)
            return 2
        fmt_name = {"q8_0": "Q8_0", "q4_0": "Q4_0", "q4k": "Q4_K", "q6k": "Q6_K"}[m.group(1)]
        rows, cols, n = int(m.group(2)), int(m.group(3)), int(m.group(4))
    fmt = B.FORMATS[fmt_name]
    K, W = max(1, args.steps), max(0, args.warmup)

    wire = synth_weight(fmt, rows, cols, args.seed)
    x = np.random.default_rng(args.seed + 1).standard_normal((n, cols)).astype(np.float32)
    copies = args.copies or max(2, min(32, -(-600_000_000 // wire.nbytes)))
    weights = [Weight.upload(fmt, rows, cols, wire) for _ in range(copies)]
    alg_bytes = wire.nbytes + 4 * cols * n + 4 * rows * n

    stream = C.c_void_p()
    check(L.cml_stream_create(C.byref(stream)))
    xd = DeviceBuffer.from_numpy(x)
    ws_bytes = L.cml_matmul_workspace_bytes(fmt, cols, n)
    ws = DeviceBuffer(ws_bytes)
    out = DeviceBuffer(n * rows * 4)
    timer = Timer(stream)

    def step(i):
        check(L.cml_matmul_f32(weights[i % copies].handle, xd.ptr, n, out.ptr, ws.ptr, ws_bytes, stream), "cml_matmul_f32")

    # warm-up (eager), then the timed region: exactly K steps replayed from one graph
    for i in range(W):
        step(i)
    check(L.cml_stream_sync(stream))
    # steps K.  A replay of few steps is shorter than the GPU's clock ramp, so the graph is first
    # replayed untimed, then several replays are timed and the median replay is reported.
    timers = [timer] + [Timer(stream) for _ in range(63)]
    ms_per_step, ms_total, const_ms, replays = steps_ms(stream, step, K, timers)
    replay_overhead_us = const_ms * 1e3
    # the same K steps launched one by one from Python, for the record
    check(L.cml_stream_sync(stream))
    eager_us = None
    if not args.cold_only:
        t0 = time.perf_counter()
        for i in range(K):
            step(i)
        check(L.cml_stream_sync(stream))
        eager_us = (time.perf_counter() - t0) / K * 1e6

    # dominant kernel alone: the gemv/gemm on already quantized activations
    per = 256 if fmt_name in ("Q4_K", "Q6_K") else 32
    qd = DeviceBuffer(n * cols)
    sd = DeviceBuffer(n * (cols // per) * 4)
    quant = L.cml_quantize_q8_k if per == 256 else L.cml_quantize_q8_0
    check(quant(xd.ptr, n, cols, qd.ptr, sd.ptr, stream))

    # Decode at the usual hidden sizes runs quantize + matvec as ONE kernel (Q4_K up to 4096 values
    # per row, Q8_0 / Q4_0 up to 8192 values and 32768 rows): there the step itself is the dominant kernel's launch.
    # Elsewhere it is the matvec on quantized activations.
    # The library's launch counters say which it is: one launch per step = the step is the dominant kernel's launch.
    launches_before, report_before = L.cml_kernel_launches(b""), launch_report()
    step(0)
    launches_per_step = int(L.cml_kernel_launches(b"") - launches_before)
    report_after = launch_report()
    kernels_of_step = sorted(k for k, v in report_after.items() if v > report_before.get(k, 0))
    fused = launches_per_step == 1   # one, two or a few tokens quantized inside the matvec launch

    def gemv_cold(i):
        if fused:
            step(i)
        else:
            check(L.cml_gemm(weights[i % copies].handle, qd.ptr, sd.ptr, n, out.ptr, stream), "cml_gemm")

    def gemv_warm(i):
        if fused:
            check(L.cml_matmul_f32(weights[0].handle, xd.ptr, n, out.ptr, ws.ptr, ws_bytes, stream), "cml_matmul_f32")
        else:
            check(L.cml_gemm(weights[0].handle, qd.ptr, sd.ptr, n, out.ptr, stream), "cml_gemm")

    def per_step(fn):
        return steps_ms(stream, fn, K, timers)[0]

    kern_ms = per_step(gemv_cold)
    # where the step quantizes in the kernel: the same matvec on an activation quantized ONCE beforehand,
    # the way the reference shares one quantized activation between the projections that read it
    # (SharedActivation, src/gemma4_runtime.rs:1288-1340) -- what a second projection of the same input costs
    shared_ms = None
    if fused and not args.cold_only:
        shared_ms = per_step(lambda i: check(L.cml_gemm(weights[i % copies].handle, qd.ptr, sd.ptr, n, out.ptr, stream), "cml_gemm"))
    warm_ms = None
    if not args.cold_only:
        warm_ms = per_step(gemv_warm)
    # what the SHAPE allows a single launch: the matvec's own loads with nothing behind them (Q4_K),
    # and the best of a few read-only launches over the same number of bytes
    ceiling = None
    if n == 1 and not args.cold_only:
        ceiling = {}
        if fmt_name == "Q4_K":
            scratch = DeviceBuffer(16)

            def loads_only(i):
                check(L.cml_calibrate_weight_loads(weights[i % copies].handle, scratch.ptr, stream), "cml_calibrate_weight_loads")

            ceiling["matvec_loads_only_us"] = round(per_step(loads_only) * 1e3, 3)
            # the same launch with one part taken out at a time (shapes the eight-wave launch serves): what the
            # activation prologue and the output store each cost
            rc_probe = L.cml_calibrate_matvec_ablation(weights[0].handle, xd.ptr, out.ptr, 1, stream)
            if rc_probe == 0:
                for key, mask in (("matvec_without_activation_us", 1), ("matvec_without_store_us", 4)):
                    def ablated(i, mask=mask):
                        check(L.cml_calibrate_matvec_ablation(weights[i % copies].handle, xd.ptr, out.ptr, mask, stream),
                              "cml_calibrate_matvec_ablation")
                    ceiling[key] = round(per_step(ablated) * 1e3, 3)
                step(0)  # a real result back into `out`
        best_us, bufs = None, None
        for groups, in_flight in ((2048, 4), (4096, 4), (8192, 4), (2048, 8)):
            us, bufs = time_read_only(stream, timers, wire.nbytes // 16 * 16, K, in_flight, groups, bufs)
            best_us = us if best_us is None else min(best_us, us)
        del bufs
        ceiling["read_only_us"] = round(best_us, 3)
        floor_us = min(ceiling[k] for k in ("matvec_loads_only_us", "read_only_us") if k in ceiling)
        ceiling["us_per_launch"] = floor_us
        ceiling["gbs"] = round(alg_bytes / floor_us / 1e3, 2)
        ceiling["frac"] = round(alg_bytes / floor_us / 1e3 / HBM_PEAK_GBS, 4)
        ceiling["note"] = ("launches that only read this weight's bytes (the matvec's own load instructions with nothing "
                           "behind them; the best of four plain grid-stride read launches), same graph replay and rotation. "
                           "Measured reference points, not bounds: for a launch of tens of MB they show how much of the "
                           "distance to the roofline the launch itself costs; on matrices of hundreds of MB the matvec's "
                           "tiled, non-temporal access pattern outruns the plain read")
    check(L.cml_stream_sync(stream))
    result = out.to_numpy(np.float32, (n, rows))
    if not np.all(np.isfinite(result)):
        print("non-finite output", file=sys.stderr)
        return 4

    achieved = alg_bytes / (kern_ms * 1e-3) / 1e9
    # the counter reading for this configuration, if one was taken and this run launched the kernel it was taken for
    traffic_bytes, traffic_source = None, None
    reading = TRAFFIC_READINGS.get(args.config)
    if reading is not None:
        if any(k.startswith(reading[1]) for k in kernels_of_step) or any(k.startswith(reading[1]) for k in launch_report()):
            traffic_bytes = reading[0]
            traffic_source = {"file": TRAFFIC_SOURCE, "kernel": reading[2], "counters": "FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 (copy-kernel yardstick), KiB per dispatch"}
        else:
            traffic_source = {"file": TRAFFIC_SOURCE, "kernel": reading[2], "note": "reading not applied: this run launched other kernels"}
    line = {
        "metric": "Q4_K matvec µs + achieved HBM GB/s (% of peak), 14336x4096, batch 1"
                  if args.config == "q4k_14336x4096_n1" else f"{fmt_name} matvec µs + achieved HBM GB/s, {rows}x{cols}, batch {n}",
        "value": round(alg_bytes / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 6),
        "us_per_call": round(ms_per_step * 1e3, 3),
        "pct_of_hbm_peak": round(100.0 * alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.config, "format": fmt_name, "rows": rows, "cols": cols, "tokens": n,
                   "algorithmic_bytes_per_call": alg_bytes, "weight_copies_rotated": copies,
                   "step": "quantize activation + fused dequantize-matvec (cml_matmul_f32), graph replay",
                   "launches_per_step": launches_per_step,
                   "kernels": kernels_of_step,
                   "replays": replays,
                   "timing": f"a graph of {K} steps replayed untimed for {SETTLE_MS:.0f} ms of GPU time, then {replays} replays timed back "
                             "to back between their own HIP events; ms_per_step = (median replay - launch constant) / K, the "
                             f"constant a replay pays for being launched measured as 2 T(k) - T(2k) on graphs of k = {min(K, LAUNCH_CAL_STEPS)} "
                             "and 2k steps (for K <= 64 that is (T(2K) - T(K)) / K)",
                   "replay_launch_overhead_us": round(replay_overhead_us, 3),
                   "k_step_replay_ms": round(ms_total, 6),
                   "raw_us_per_step": round(ms_total / K * 1e3, 3),   # the K-step replay divided by K, nothing taken off
                   "eager_python_us_per_call": None if eager_us is None else round(eager_us, 3)},
        "roofline": {"bound": "hbm",
                     "kernel": f"gemv_{fmt_name.lower()} with the activation quantizer fused in (cml_matmul_f32, one launch)" if fused
                     else f"gemv_{fmt_name.lower()} (cml_gemm on quantized activations)",
                     "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_bytes, "traffic_source": traffic_source,
                     "us_per_launch": round(kern_ms * 1e3, 3),
                     "rocprofv3": rocprof_summary(args.config, kernels_of_step),
                     "cache_warm_us_per_launch": None if warm_ms is None else round(warm_ms * 1e3, 3),
                     "cache_warm_gbs": None if warm_ms is None else round(alg_bytes / (warm_ms * 1e-3) / 1e9, 2),
                     "shared_activation_us_per_launch": None if shared_ms is None else round(shared_ms * 1e3, 3),
                     "shape_ceiling": ceiling},
    }
    if n >= 8:
        # the batched shapes also have a matrix-core side: 2*rows*cols*tokens integer operations
        tops = 2.0 * rows * cols * n / (kern_ms * 1e-3) / 1e12
        line["roofline"]["mfma"] = {"achieved": round(tops, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                    "frac": round(tops / INT8_PEAK_TOPS, 4)}
    if args.cpu_seconds > 0:
        line["cpu_baseline"] = cpu_baseline(fmt, wire, rows, cols, x, alg_bytes, args.cpu_seconds)
    print(json.dumps(line, ensure_ascii=False))
    return 0


if __name__ == "__main__":
    sys.exit(main())
