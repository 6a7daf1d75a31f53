#!/usr/bin/env python3
"""Benchmark of the block-quantized weight path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  The default workload is the configuration the headline metric is quoted on:
Q4_K batch-1 decode GEMV, W 14336x4096, x bf16, fp32 accumulate.  A step is one pass of that GEMV
over a batch of 16 distinct weight tensors (16 same-shaped layers of a decode step): 16 x 33 MB is
larger than the 256 MB last-level cache, so every step streams its weights from HBM.

Timing: HIP events recorded on the stream the kernels are launched on (the null stream, or the stream of a recorded
launch sequence that is replayed), bracketed by
stream synchronisation; inputs are resident in HBM before the timed region.  `roofline.achieved` is
algorithmic bytes (or flops) per launch divided by the average launch duration over the timed region.
The CPU baseline is the oracle's restatement of the reference algorithm (dequantize, then an f32
dot product) on a bounded sample of the same workload: `value` on one thread, as the reference runs
it, and `all_cores` with the rows / blocks spread over every host thread; `host` names the machine.

The default invocation also times the other two parts of the headline metric (the Q4_K GEMM at M = 512 and
the f32 -> Q4_K_M quantizer) and a plain read of the same bytes, and reports them under `extra`.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
# HBM bytes per launch as recorded from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled against a streaming kernel
# of known size; constants taken from the profile summaries named here, not measured by this script
RECORDED_TRAFFIC = {"gemv_q4k_14336x4096": (33287193, "profiles/qgemv_q4k_14336x4096.md"),
                    "gemv_q4k_4096x14336": (33414162, "profiles/qgemv_q4k_4096x14336.md"),
                    "gemv_q6k_14336x4096": (48532488, "profiles/qgemv_other_types.md"),
                    "gemv_q8_0_14336x4096": (62653287, "profiles/qgemv_other_types.md"),
                    "gemv_q5k_6144x4096": (17530063, "profiles/qgemv_other_types.md"),
                    "gemv_q3k_14336x4096": (25568799, "profiles/qgemv_other_types.md"),
                    "gemv_q2k_14336x4096": (19580687, "profiles/qgemv_other_types.md"),
                    # per call: pre-pass + matrix kernel; per step: all 226 tensors; per tensor
                    "gemm_q4k_m512": (99287040, "profiles/qgemm_q4k_m512.md"),
                    "quantize_llama3_8b_q4km": (37284068260, "profiles/quantize_q4km_llama3_8b.md"),
                    "dequantize_14336x4096": (268075008, "profiles/dequantize_14336x4096.md")}
BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16/fp16 MFMA, published
Q8_0, Q4K, Q6K = 8, 12, 14


def load():
    import pmetal_amd as pm
    from pmetal_amd import _lib
    lib = _lib.load()  # raises if the HIP library is missing: there is no fallback
    pm.init(0)
    return pm, _lib, lib


class Timer:
    def __init__(self, pm, lib):
        self.pm, self.lib = pm, lib
        self.e0, self.e1 = lib.pmetal_hip_event_create(), lib.pmetal_hip_event_create()
        self.stream = None  # the stream fn() launches on: the events are recorded there

    def run(self, fn, steps, warmup):
        """W untimed + exactly K timed calls of fn(); returns (event_ms, wall_ms)."""
        pm, lib, st = self.pm, self.lib, self.stream
        for _ in range(warmup):
            fn()
        pm.check(lib.pmetal_hip_sync(st))
        t0 = time.perf_counter()
        pm.check(lib.pmetal_hip_event_record(self.e0, st))
        for _ in range(steps):
            fn()
        pm.check(lib.pmetal_hip_event_record(self.e1, st))
        ms = C.c_float()
        pm.check(lib.pmetal_hip_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        pm.check(lib.pmetal_hip_sync(st))
        return float(ms.value), (time.perf_counter() - t0) * 1e3


def device_weights(pm, lib, t, n_elems, seed, outlier_rate=0.0):
    """Random-init N(0, 0.02) tensor generated on the device and quantized there; returns the packed buffer."""
    f = pm.DeviceBuffer(4 * n_elems)
    pm.check(lib.pmetal_hip_fill_normal_f32(f.ptr, n_elems, seed, 0.02, outlier_rate, 0.5, None))
    nbytes = lib.pmetal_hip_tensor_size(t, n_elems)
    q = pm.DeviceBuffer(nbytes)
    pm.check(lib.pmetal_hip_quantize_dev(t, f.ptr, n_elems, q.ptr, nbytes, None), "quantize")
    pm.check(lib.pmetal_hip_sync(None))
    f.free()
    return q


def bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def gemv_bytes(t, n, k, x_bytes):
    per_block = {Q8_0: (34, 32), Q4K: (144, 256), Q6K: (210, 256), 13: (176, 256), 11: (110, 256), 10: (84, 256)}[t]
    return n * (k // per_block[1]) * per_block[0] + k * x_bytes + n * 4


def host_description():
    """Logical CPUs of the host, the CPUs this process may use, and the CPU model."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"nproc": os.cpu_count() or 1, "usable_cpus": usable, "cpu_model": model}


def baseline_threads():
    """Threads of the all-cores leg: the CPUs this process may use, at most 64."""
    return max(1, min(host_description()["usable_cpus"], 64))


def timed_reps(fn, budget_s):
    reps, t0 = 0, time.perf_counter()
    while reps == 0 or time.perf_counter() - t0 < budget_s:
        fn()
        reps += 1
    return reps, time.perf_counter() - t0


def cpu_baseline_gemv(t, n, k, budget_s=6.0):
    """Oracle: reference dequantize + sequential f32 dot, one thread, on whole rows of the same shape."""
    from oracle import binding as oracle
    oracle.build()
    rows = min(n, 2048)
    rng = np.random.default_rng(5)
    w = (rng.standard_normal(rows * k) * 0.02).astype(np.float32)
    wq = oracle.quantize(t, w)
    x = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32)))
    oracle.qmatvec(t, wq, rows, k, x, acc="f32")
    reps, dt = timed_reps(lambda: oracle.qmatvec(t, wq, rows, k, x, acc="f32"), budget_s)
    gbs = gemv_bytes(t, rows, k, 2) * reps / dt / 1e9
    th = baseline_threads()
    reps_mt, dt_mt = timed_reps(lambda: oracle.qmatvec(t, wq, rows, k, x, acc="f32", threads=th), budget_s / 2)
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x (dequantize + f32 matvec) of {rows}x{k} rows of the same shape, {dt:.1f} s",
            "all_cores": {"value": round(gemv_bytes(t, rows, k, 2) * reps_mt / dt_mt / 1e9, 3), "unit": "GB/s", "cores": th,
                          "sample": f"{reps_mt} x the same rows spread over {th} threads, {dt_mt:.1f} s"},
            "host": host_description()}


def cpu_baseline_quantize(budget_s=6.0):
    """Oracle: the reference's quantizers, one thread, on f32 tensors in the model's Q4_K : Q6_K element ratio."""
    from oracle import binding as oracle
    oracle.build()
    rng = np.random.default_rng(6)
    x4 = (rng.standard_normal(3 << 18) * 0.02).astype(np.float32)   # 786432 elements to Q4_K
    x6 = (rng.standard_normal(1 << 18) * 0.02).astype(np.float32)   # 262144 elements to Q6_K (the recipe's 26 %)
    oracle.quantize(Q4K, x4[:4096]), oracle.quantize(Q6K, x6[:4096])

    def once(threads=1):
        oracle.quantize(Q4K, x4, threads=threads)
        oracle.quantize(Q6K, x6, threads=threads)

    reps, dt = timed_reps(once, budget_s)
    th = baseline_threads()
    reps_mt, dt_mt = timed_reps(lambda: once(th), budget_s / 2)
    return {"value": round(4.0 * (x4.size + x6.size) * reps / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x (786432 elements to Q4_K + 262144 to Q6_K), {dt:.1f} s",
            "all_cores": {"value": round(4.0 * (x4.size + x6.size) * reps_mt / dt_mt / 1e9, 4), "unit": "GB/s", "cores": th,
                          "sample": f"{reps_mt} x the same elements, super-block ranges spread over {th} threads, {dt_mt:.1f} s"},
            "host": host_description()}


def cpu_baseline_dequantize(budget_s=10.0):
    """Oracle: the reference's dequantize_q4k, one thread."""
    from oracle import binding as oracle
    oracle.build()
    n = 1 << 22
    wq = oracle.quantize(Q4K, (np.random.default_rng(9).standard_normal(n) * 0.02).astype(np.float32))
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        oracle.dequantize(Q4K, wq, [n])
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": round((wq.size + 4.0 * n) * reps / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x dequantize of {n} Q4_K elements, {dt:.1f} s"}


def cpu_baseline_gemm(t, m, n, k, budget_s=6.0):
    """Oracle: reference dequantize + f32 matmul (row by row, sequential dot products), one thread, on a slice."""
    from oracle import binding as oracle
    oracle.build()
    rows, mm = min(n, 256), min(m, 64)
    rng = np.random.default_rng(7)
    wq = oracle.quantize(t, (rng.standard_normal(rows * k) * 0.02).astype(np.float32))
    x = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(rng.standard_normal(mm * k).astype(np.float32))).reshape(mm, k)
    oracle.qmatmul(t, wq, rows, k, x[:1])
    reps, dt = timed_reps(lambda: oracle.qmatmul(t, wq, rows, k, x), budget_s)
    th = baseline_threads()
    reps_mt, dt_mt = timed_reps(lambda: oracle.qmatmul(t, wq, rows, k, x, threads=th), budget_s / 2)
    return {"value": round(2.0 * mm * rows * k * reps / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x (dequantize + matmul) of {mm} x {rows} x {k}, {dt:.1f} s",
            "all_cores": {"value": round(2.0 * mm * rows * k * reps_mt / dt_mt / 1e12, 6), "unit": "TFLOP/s", "cores": th,
                          "sample": f"{reps_mt} x the same product, weight rows spread over {th} threads, {dt_mt:.1f} s"},
            "host": host_description()}


def cpu_baseline_decode(pm, model="qwen3_0.6b", budget_s=15.0):
    """Oracle: dequantize + f32 matvec, one thread, over the projections of the first two layers of the stack (the first
    layer's attention projections for the 8B shape, whose single layers take seconds on one core)."""
    from oracle import binding as oracle
    oracle.build()
    all_lins = qwen3_06b_linears(pm) if model == "qwen3_0.6b" else llama3_8b_linears(pm)
    prefixes = ("blk.0.", "blk.1.") if model == "qwen3_0.6b" else ("blk.0.attn",)
    lins = [l for l in all_lins if l[0].startswith(prefixes)]
    rng = np.random.default_rng(8)
    ws = [(t, oracle.quantize(t, (rng.standard_normal(n * k) * 0.02).astype(np.float32)), n, k) for _, n, k, t in lins]
    xs = {k: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))) for k in sorted({l[2] for l in lins})}
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        for t, wq, n, k in ws:
            oracle.qmatvec(t, wq, n, k, xs[k], acc="f32")
        reps += 1
    dt = time.perf_counter() - t0
    sample_bytes = sum(gemv_bytes(t, n, k, 2) for t, _, n, k in ws)
    total_bytes = sum(gemv_bytes(t, n, k, 2) for _, n, k, t in all_lins)
    return {"value": round(reps / dt * sample_bytes / total_bytes, 4), "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x the {len(ws)} projections {' / '.join(prefixes)}* ({sample_bytes} of {total_bytes} weight bytes per token), "
                      f"scaled by bytes, {dt:.1f} s"}


def bench_gemv(args, n, k, t=Q4K, copies=16, passes=8):
    """One step = `passes` sweeps over `copies` distinct weight tensors, one GEMV launch per tensor."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    ws = [device_weights(pm, lib, t, n * k, 1000 + i) for i in range(copies)]
    x = pm.DeviceBuffer.from_host(bf16_bits(np.random.default_rng(1).standard_normal(k)))
    ys = [pm.DeviceBuffer(4 * n) for _ in range(copies)]
    descs = (_lib.LinearDesc * copies)()
    for i in range(copies):
        descs[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, ws[i].ptr, x.ptr, ys[i].ptr)

    # One launch per matrix: consecutive descriptors name different (identical) activation buffers, because the batch entry
    # point sends consecutive matrices that share x two to a launch where the kernel allows it.
    x2 = pm.DeviceBuffer.from_host(bf16_bits(np.random.default_rng(1).standard_normal(k)))
    solo = (_lib.LinearDesc * copies)()
    for i in range(copies):
        solo[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, ws[i].ptr, (x if i % 2 == 0 else x2).ptr, ys[i].ptr)

    def sweeps(descs_):
        def run():
            for _ in range(passes):
                pm.check(lib.pmetal_hip_qgemv_batch(descs_, copies, None))
        return run

    eager_ms, _ = timer.run(sweeps(solo), args.steps, args.warmup)
    launches = args.steps * copies * passes
    # the same launches recorded once (a HIP graph) and replayed with one submission per step: what a decoder does
    stream = lib.pmetal_hip_stream_create()
    pm.check(lib.pmetal_hip_record_begin(stream))
    for _ in range(passes):
        pm.check(lib.pmetal_hip_qgemv_batch(solo, copies, stream))
    rec = lib.pmetal_hip_record_end(stream)
    if not rec:
        raise RuntimeError(lib.pmetal_hip_last_error_message())
    timer.stream = stream
    ev_ms, wall_ms = timer.run(lambda: pm.check(lib.pmetal_hip_replay(rec, stream)), args.steps, args.warmup)
    timer.stream = None
    pm.check(lib.pmetal_hip_recording_destroy(rec))
    bytes_per_launch = gemv_bytes(t, n, k, 2)
    us_per_launch = ev_ms * 1e3 / launches
    gbs = bytes_per_launch / (us_per_launch * 1e-6) / 1e9

    # same kernel with one weight tensor re-read from the last-level cache (reported, never `value`)
    one = (_lib.LinearDesc * copies)()
    for i in range(copies):
        one[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, ws[0].ptr, (x if i % 2 == 0 else x2).ptr, ys[0].ptr)
    c_ms, _ = timer.run(sweeps(one), args.steps, args.warmup)
    cached_gbs = bytes_per_launch / (c_ms * 1e-3 / launches) / 1e9
    # all sixteen sharing one x (as gate / up do): two matrices per launch where the kernel allows it
    b_ms, _ = timer.run(sweeps(descs), args.steps, args.warmup)
    # what a launch that only reads the same weight bytes takes on this machine, from HBM and from the cache
    sink = pm.DeviceBuffer(16)
    w_bytes = lib.pmetal_hip_tensor_size(t, n * k)

    def reads(bufs):
        def run():
            for _ in range(passes):
                for b in bufs:
                    pm.check(lib.pmetal_hip_read_probe(b.ptr, w_bytes, sink.ptr, None))
        return run

    r_ms, _ = timer.run(reads(ws), args.steps, args.warmup)
    rc_ms, _ = timer.run(reads([ws[0]] * copies), args.steps, args.warmup)
    read_us, read_cached_us = r_ms * 1e3 / launches, rc_ms * 1e3 / launches
    return {
        "value": gbs, "ms_per_step": wall_ms / args.steps, "event_ms_per_step": ev_ms / args.steps,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": {Q4K: "k_qgemv_q4k_rows" if k in (2048, 4096) else "k_qgemv_q4k_chunk", Q6K: "k_qgemv_q6k_chunk", Q8_0: "k_qgemv_q8_0_chunk", 13: "k_qgemv_q5k_chunk", 11: "k_qgemv_q23k_chunk<FormatQ3K>", 10: "k_qgemv_q23k_chunk<FormatQ2K>"}[t], "bytes_per_launch": bytes_per_launch,
                     "us_per_launch": round(us_per_launch, 3)},
        "extra": {"submission": "the step's 128 launches recorded once and replayed (one submission per step)",
                  "eager_us_per_launch": round(eager_ms * 1e3 / launches, 3),
                  "cache_resident_GBps": round(cached_gbs, 1), "cache_resident_us_per_launch": round(c_ms * 1e3 / launches, 3),
                  "weight_copies": copies, "launches_per_step": copies * passes,
                  "batch_entry_us_per_matrix": round(b_ms * 1e3 / launches, 3),
                  "plain_read_us": {"hbm": round(read_us, 3), "cache_resident": round(read_cached_us, 3),
                                    "bytes": w_bytes, "hbm_GBps": round(w_bytes / (read_us * 1e-6) / 1e9, 1),
                                    "what": "pmetal_hip_read_probe over the same weight tensors, same launch pattern: a kernel that only reads"},
                  "gemv_over_plain_read": round(us_per_launch / read_us, 3)},
    }, (t, n, k)


def bench_gemv_q8k(args, n, k, t=Q4K, copies=16):
    """One step = `copies` x (quantize the f32 activations to Q8_K, integer-dot GEMV), weights rotating through HBM."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    ws = [device_weights(pm, lib, t, n * k, 1000 + i) for i in range(copies)]
    x = pm.DeviceBuffer.from_host(np.random.default_rng(1).standard_normal(k).astype(np.float32))
    xq = pm.DeviceBuffer(lib.pmetal_hip_q8k_size(k))
    ys = [pm.DeviceBuffer(4 * n) for _ in range(copies)]

    def step():
        for i in range(copies):
            pm.check(lib.pmetal_hip_quantize_q8k_dev(x.ptr, k, xq.ptr, lib.pmetal_hip_q8k_size(k), None))
            pm.check(lib.pmetal_hip_qgemv_q8k(t, ws[i].ptr, n, k, xq.ptr, ys[i].ptr, None))

    def gemv_only():
        for i in range(copies):
            pm.check(lib.pmetal_hip_qgemv_q8k(t, ws[i].ptr, n, k, xq.ptr, ys[i].ptr, None))

    ev_ms, wall_ms = timer.run(step, args.steps, args.warmup)
    g_ms, _ = timer.run(gemv_only, args.steps, args.warmup)
    launches = args.steps * copies
    bytes_per_launch = pm.GgmlType(t).tensor_size(n * k) + 4 * k + lib.pmetal_hip_q8k_size(k) * 2 + 4 * n
    us = ev_ms * 1e3 / launches
    gbs = bytes_per_launch / (us * 1e-6) / 1e9
    return {
        "value": gbs, "ms_per_step": wall_ms / args.steps, "event_ms_per_step": ev_ms / args.steps,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_qgemv_q4k_q8k (+ k_quantize_q8k)" if t == Q4K else "k_qgemv_q6k_q8k (+ k_quantize_q8k)",
                     "bytes_per_launch": bytes_per_launch, "us_per_launch": round(us, 3)},
        "extra": {"gemv_only_us_per_launch": round(g_ms * 1e3 / launches, 3), "weight_copies": copies},
    }, (t, n, k)


def cpu_baseline_gemv_q8k(t, n, k, budget_s=12.0):
    """Oracle: quantize_q8k of the activations + the scalar vec_dot over every row, one thread, on a slice of the rows."""
    from oracle import binding as oracle
    oracle.build()
    rows = min(n, 2048)
    rng = np.random.default_rng(7)
    wq = oracle.quantize(t, (rng.standard_normal(rows * k) * 0.02).astype(np.float32))
    x = rng.standard_normal(k).astype(np.float32)
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        oracle.qmatvec_q8k(t, wq, rows, k, oracle.quantize_q8k(x))
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": round(reps * wq.size / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x (quantize_q8k + vec_dot over {rows}x{k} rows of the same shape), {dt:.1f} s"}


def bench_calibrate(args, n, k):
    """One step = the round trips of calibrate_tensor for one resident 14336 x 4096 f32 tensor: for each candidate type
    of the reference's default list (Q8_K, Q6_K, Q5_K, Q4_K, Q3_K, Q2_K) quantize, then dequantize and score in one pass."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    ne = n * k
    x = pm.DeviceBuffer(4 * ne)
    pm.check(lib.pmetal_hip_fill_normal_f32(x.ptr, ne, 11, 0.02, 1e-3, 0.5, None))
    cands = [15, 14, 13, 12, 11, 10]
    qs = {t: pm.DeviceBuffer(lib.pmetal_hip_tensor_size(t, ne)) for t in cands}
    scores = {}
    import ctypes as C

    def step():
        for t in cands:
            nb = lib.pmetal_hip_tensor_size(t, ne)
            pm.check(lib.pmetal_hip_quantize_dev(t, x.ptr, ne, qs[t].ptr, nb, None))
            sc = C.c_double()
            pm.check(lib.pmetal_hip_kl_divergence_quantized_dev(t, qs[t].ptr, nb, x.ptr, ne, 1, C.byref(sc), None))
            scores[t] = sc.value

    steps, warm = max(1, args.steps // 20), max(1, args.warmup // 10)
    ev_ms, wall_ms = timer.run(step, steps, warm)
    # per candidate: quantize reads 4n and writes the blocks, the fused comparison reads the blocks and 4n
    bytes_per_step = sum(4 * ne + 2 * lib.pmetal_hip_tensor_size(t, ne) + 4 * ne for t in cands)
    gbs = 4.0 * ne * len(cands) / (wall_ms / steps * 1e-3) / 1e9
    res = {
        "value": gbs, "ms_per_step": wall_ms / steps, "event_ms_per_step": ev_ms / steps,
        "roofline": {"bound": "hbm", "achieved": round(bytes_per_step / (wall_ms / steps * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(bytes_per_step / (wall_ms / steps * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_quantize_* / k_kl_sums_kq", "bytes_per_step": bytes_per_step},
        "extra": {"scores": {str(t): scores[t] for t in cands}, "steps_run": steps},
    }
    args.steps, args.warmup = steps, warm
    return res, (Q4K, n, k)


def cpu_baseline_calibrate(budget_elems=1 << 20):
    """Oracle: calibrate_tensor (quantize, dequantize, score for the same six candidates), one thread, on 2^20 elements."""
    from oracle import binding as oracle
    oracle.build()
    x = (np.random.default_rng(3).standard_normal(budget_elems) * 0.02).astype(np.float32)
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 10.0:
        oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [budget_elems // 256, 256], candidates=(15, 14, 13, 12, 11, 10), order=1)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": round(4.0 * budget_elems * 6 * reps / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x calibrate_tensor over {budget_elems} elements, six candidates, {dt:.1f} s"}


def bench_gemm(args, m, n, k, t=Q4K):
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    # short batches are bound by reading the weights: rotate over enough tensors that they come from HBM, not from the
    # 256 MB last-level cache (a step is then one call per tensor)
    copies = 10 if m <= 128 else 1
    wl = [device_weights(pm, lib, t, n * k, 2000 + 10 * i) for i in range(copies)]
    w = wl[0]
    x = pm.DeviceBuffer.from_host(bf16_bits(np.random.default_rng(2).standard_normal(m * k)))
    y = pm.DeviceBuffer(2 * m * n)

    def per_call():
        for wi in wl:
            pm.check(lib.pmetal_hip_qgemm(t, wi.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_BF16, 0, None))

    step, reblocked_us = per_call, None
    rb_bytes = lib.pmetal_hip_reblock_size(t, n, k)
    if rb_bytes:  # Q5_K / Q3_K / Q2_K have matrix kernels of their own; the re-blocked form (one or two Q6_K tensors) is timed beside them
        rb = pm.DeviceBuffer(rb_bytes)
        pm.check(lib.pmetal_hip_reblock_dev(t, w.ptr, n, k, 0, rb.ptr, rb_bytes, None), "reblock")
        rb_ms, _ = timer.run(lambda: pm.check(lib.pmetal_hip_qgemm_reblocked(t, rb.ptr, rb_bytes, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_BF16, None)),
                             args.steps, args.warmup)
        reblocked_us = rb_ms * 1e3 / args.steps
        rb.free()
    ev_ms, wall_ms = timer.run(step, args.steps, args.warmup)
    eager_us = ev_ms * 1e3 / (args.steps * copies)
    submission, replay_us = "one call after the other (eager launches)", None
    if step is per_call:
        # the same calls recorded once (a HIP graph of eight passes) and replayed with one submission per step, as a prefill
        # that runs its projections from a recording submits them; the eager figure stays in `extra`
        reps = 8
        stream = lib.pmetal_hip_stream_create()
        for wi in wl:  # (the library's scratch for this stream exists before the recording starts)
            pm.check(lib.pmetal_hip_qgemm(t, wi.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_BF16, 0, stream))
        pm.check(lib.pmetal_hip_sync(stream))
        pm.check(lib.pmetal_hip_record_begin(stream))
        for _ in range(reps):
            for wi in wl:
                pm.check(lib.pmetal_hip_qgemm(t, wi.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_BF16, 0, stream))
        rec = lib.pmetal_hip_record_end(stream)
        if not rec:
            raise RuntimeError(lib.pmetal_hip_last_error_message())
        timer.stream = stream
        r_steps = max(args.steps // reps, 3)
        r_ev, r_wall = timer.run(lambda: pm.check(lib.pmetal_hip_replay(rec, stream)), r_steps, max(args.warmup // reps, 1))
        timer.stream = None
        pm.check(lib.pmetal_hip_recording_destroy(rec))
        pm.check(lib.pmetal_hip_stream_destroy(stream))
        replay_us = r_ev * 1e3 / (r_steps * reps * copies)
        if replay_us < eager_us:  # (`value` is the faster of the two ways to submit the same calls; both figures are in `extra`)
            ev_ms, wall_ms = r_ev * args.steps / (r_steps * reps), r_wall * args.steps / (r_steps * reps)
            submission = f"{reps} passes over the weights recorded once and replayed (one submission per {reps * copies} calls)"
    # what the matrix cores of this machine sustain in a register-only MFMA loop (no memory, no LDS) of about the
    # same length, with operands that vary: the ceiling any kernel here works under (the published peak assumes
    # the top clock, which a matrix loop does not hold)
    sink = pm.DeviceBuffer(4)
    probe_iters = 20000
    p_ms, _ = timer.run(lambda: pm.check(lib.pmetal_hip_mfma_probe_f16(probe_iters, 1, 256, sink.ptr, None)), 3, 1)
    sustained = 3 * 256 * 8 * probe_iters * 4 * 32768.0 / (p_ms * 1e-3) / 1e12
    flops = 2.0 * m * n * k
    us = ev_ms * 1e3 / (args.steps * copies)
    tflops = flops / (us * 1e-6) / 1e12
    dense = dense_library_tflops(m, n, k) if args.dense_library else None
    pair_us = None
    if t in (Q4K, Q6K, Q8_0, 13, 11, 10):  # two weights against the same activations (gate / up): one pre-pass for both
        if copies == 1:
            wl.append(device_weights(pm, lib, t, n * k, 2001))
        y2 = pm.DeviceBuffer(2 * m * n)
        pairs = [(_lib.GemmDesc * 2)(_lib.GemmDesc(t, pm.DTYPE_BF16, 0, 0, n, wl[i].ptr, y.ptr), _lib.GemmDesc(t, pm.DTYPE_BF16, 0, 0, n, wl[i + 1].ptr, y2.ptr))
                 for i in range(0, len(wl) - 1, 2)]

        def batched():
            for d in pairs:
                pm.check(lib.pmetal_hip_qgemm_batch(d, 2, k, x.ptr, pm.DTYPE_BF16, m, None))

        b_ms, _ = timer.run(batched, args.steps, args.warmup)
        pair_us = b_ms * 1e3 / args.steps / (2 * len(pairs))
    # independent calls (each with its own pre-pass) on three streams of the host's own: one call's pre-pass, first and last
    # workgroups overlap the others' matrix kernels.  A throughput figure for callers that have independent GEMMs; not `value`.
    streams = [lib.pmetal_hip_stream_create() for _ in range(3)]
    ys = [pm.DeviceBuffer(2 * m * n) for _ in range(3)]
    wl3 = wl if len(wl) >= 3 else wl + [device_weights(pm, lib, t, n * k, 2002 + i) for i in range(3 - len(wl))]

    def on_streams():
        for i, wi in enumerate(wl3):
            pm.check(lib.pmetal_hip_qgemm(t, wi.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, ys[i % 3].ptr, pm.DTYPE_BF16, 0, streams[i % 3]))

    for _ in range(3):
        on_streams()
    for st in streams:
        pm.check(lib.pmetal_hip_sync(st))
    reps3 = max(args.steps // 2, 5)
    t0 = time.perf_counter()
    for _ in range(reps3):
        on_streams()
    for st in streams:
        pm.check(lib.pmetal_hip_sync(st))
    streams_us = (time.perf_counter() - t0) * 1e6 / (reps3 * len(wl3))
    for st in streams:
        pm.check(lib.pmetal_hip_stream_destroy(st))
    return {
        "value": tflops, "ms_per_step": wall_ms / args.steps, "event_ms_per_step": ev_ms / args.steps,
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": ({Q4K: "k_qgemm_small", 13: "k_qgemm_small<FMT = 1>", Q6K: "k_qgemm_small_q6", Q8_0: "k_qgemm_small_q8",
                                 11: "k_qgemm_small16<Q3_K>", 10: "k_qgemm_small16<Q2_K>"}[t] + " (+ k_prep_rw)"
                                if m <= 16 else
                                {Q4K: "k_qgemm_rw", 13: "k_qgemm_rw<FMT = 1>", Q6K: "k_qgemm_rw_q6", Q8_0: "k_qgemm_rw_q8", 11: "k_qgemm_rw16<Q3_K>", 10: "k_qgemm_rw16<Q2_K>"}[t]
                                + " (+ k_prep_rw, k_rw_reduce when K is split)"),
                     "flops_per_launch": flops, "us_per_launch": round(us, 3)},
        "extra": {"calls_per_step": copies, "submission": submission, "eager_us_per_call": round(eager_us, 3),
                  "replayed_us_per_call": None if replay_us is None else round(replay_us, 3), "weights": f"{copies} tensor(s) in turn" + (" (from HBM)" if copies > 1 else " (one tensor: stays in the last-level cache)"),
                  "mfma_loop_sustained_TFLOPs": round(sustained, 1), "frac_of_sustained": round(tflops / sustained, 4),
                  "dense_library_TFLOPs": dense,
                  "two_weights_sharing_x_us_per_weight": None if pair_us is None else round(pair_us, 3),
                  "two_weights_sharing_x_TFLOPs": None if pair_us is None else round(flops / (pair_us * 1e-6) / 1e12, 1),
                  "independent_calls_on_three_streams_us_per_call": round(streams_us, 3),
                  "independent_calls_on_three_streams_TFLOPs": round(flops / (streams_us * 1e-6) / 1e12, 1),
                  **({} if reblocked_us is None else {"reblocked_form_us": round(reblocked_us, 3), "reblocked_bytes": rb_bytes})},
    }, (t, n, k)


_DENSE_SCRIPT = """
import sys, torch
m, n, k, reps = (int(a) for a in sys.argv[1:5])
x = torch.randn(m, k, device="cuda", dtype=torch.float16)
w = (torch.randn(n, k, device="cuda", dtype=torch.float32) * 0.02).to(torch.float16)
for _ in range(5):
    y = x @ w.t()
torch.cuda.synchronize()
e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
e0.record()
for _ in range(reps):
    y = x @ w.t()
e1.record()
torch.cuda.synchronize()
print("TFLOPS", 2.0 * m * n * k * reps / (e0.elapsed_time(e1) * 1e-3) / 1e12)
"""


def dense_library_tflops(m, n, k, reps=50):
    """A yardstick beside the kernel, never part of it: the f16 product of the same shape (X[m,k] W[n,k]^T, dense, already
    dequantized) through torch.matmul, i.e. the vendor's GEMM library, timed with torch's own events on this machine.  It
    runs in a child process: torch brings its own HIP runtime, which cannot share a process with the one this library loads."""
    import subprocess
    try:
        r = subprocess.run([sys.executable, "-c", _DENSE_SCRIPT, str(m), str(n), str(k), str(reps)], capture_output=True, text=True,
                           timeout=240)
    except (OSError, subprocess.TimeoutExpired):
        return None
    for line in r.stdout.splitlines():
        if line.startswith("TFLOPS"):
            return round(float(line.split()[1]), 1)
    return None


def bench_dequantize(args, n, k):
    """Blocks -> f32 of one 14336 x 4096 tensor per type; rotating over enough tensors to stay out of the last-level cache."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    out = {}
    for t, name, copies in ((Q4K, "q4k", 2), (Q6K, "q6k", 2), (Q8_0, "q8_0", 2)):
        ws = [device_weights(pm, lib, t, n * k, 4000 + i) for i in range(copies)]
        ys = [pm.DeviceBuffer(4 * n * k) for _ in range(copies)]
        nbytes = lib.pmetal_hip_tensor_size(t, n * k)

        def step():
            for w, y in zip(ws, ys):
                pm.check(lib.pmetal_hip_dequantize_dev(t, w.ptr, nbytes, y.ptr, n * k, 0, None), "dequantize")

        ev_ms, wall_ms = timer.run(step, args.steps, args.warmup)
        us = ev_ms * 1e3 / (args.steps * copies)
        out[name] = {"us_per_launch": round(us, 2), "GBps": round((nbytes + 4.0 * n * k) / (us * 1e-6) / 1e9, 1),
                     "bytes_per_launch": nbytes + 4 * n * k, "wall_ms_per_step": wall_ms / args.steps, "ev_ms_per_step": ev_ms / args.steps}
        for b in ws + ys:
            b.free()
    q = out["q4k"]
    return {
        "value": q["GBps"], "ms_per_step": q["wall_ms_per_step"], "event_ms_per_step": q["ev_ms_per_step"],
        "roofline": {"bound": "hbm", "achieved": q["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(q["GBps"] / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "k_dequantize_q4k",
                     "bytes_per_launch": q["bytes_per_launch"], "us_per_launch": q["us_per_launch"]},
        "extra": {"q6k": {k2: out["q6k"][k2] for k2 in ("us_per_launch", "GBps")},
                  "q8_0": {k2: out["q8_0"][k2] for k2 in ("us_per_launch", "GBps")}},
    }, (Q4K, n, k)


def qwen3_06b_linears(pm):
    """(gguf name, n, k, type) of every batch-1 projection of a Qwen3-0.6B-shaped decoder, Q4_K_M recipe."""
    out = []
    for layer in range(28):
        for name, n, k in (("attn_q", 2048, 1024), ("attn_k", 1024, 1024), ("attn_v", 1024, 1024),
                           ("attn_output", 1024, 2048), ("ffn_gate", 3072, 1024), ("ffn_up", 3072, 1024),
                           ("ffn_down", 1024, 3072)):
            gg = f"blk.{layer}.{name}.weight"
            out.append((gg, n, k, int(pm.q4km_tensor_type(gg, 2, 28))))
    out.append(("output.weight", 151936, 1024, int(pm.q4km_tensor_type("output.weight", 2, 28))))
    return out


def llama3_8b_tensors(pm):
    """(gguf name, n, k, type) of every quantized tensor of a Llama-3-8B-shaped model, Q4_K_M recipe."""
    out = [("token_embd.weight", 128256, 4096, int(pm.q4km_tensor_type("token_embd.weight", 2, 32)))]
    for layer in range(32):
        for name, n, k in (("attn_q", 4096, 4096), ("attn_k", 1024, 4096), ("attn_v", 1024, 4096),
                           ("attn_output", 4096, 4096), ("ffn_gate", 14336, 4096), ("ffn_up", 14336, 4096),
                           ("ffn_down", 4096, 14336)):
            gg = f"blk.{layer}.{name}.weight"
            out.append((gg, n, k, int(pm.q4km_tensor_type(gg, 2, 32))))
    out.append(("output.weight", 128256, 4096, int(pm.q4km_tensor_type("output.weight", 2, 32))))
    return out


def llama3_8b_linears(pm):
    """(gguf name, n, k, type) of every batch-1 projection of a Llama-3-8B-shaped decoder, Q4_K_M recipe."""
    return [l for l in llama3_8b_tensors(pm) if l[0] != "token_embd.weight"]


def bench_decode(args, model="qwen3_0.6b"):
    """All batch-1 linear projections of one token of a random-init decoder stack of the given shape (linears only)."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    lins = qwen3_06b_linears(pm) if model == "qwen3_0.6b" else llama3_8b_linears(pm)
    descs = (_lib.LinearDesc * len(lins))()
    keep, total_bytes = [], 0
    xs = {k: pm.DeviceBuffer.from_host(bf16_bits(np.random.default_rng(k).standard_normal(k))) for k in sorted({l[2] for l in lins})}
    for i, (name, n, k, t) in enumerate(lins):
        w = device_weights(pm, lib, t, n * k, 3000 + i)
        y = pm.DeviceBuffer(4 * n)
        keep.append((w, y))
        descs[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, w.ptr, xs[k].ptr, y.ptr)
        total_bytes += gemv_bytes(t, n, k, 2)

    def step():
        pm.check(lib.pmetal_hip_qgemv_batch(descs, len(lins), None))

    eager_ms, _ = timer.run(step, args.steps, args.warmup)
    # the same launches recorded once and replayed with one submission per token (a HIP graph)
    stream = lib.pmetal_hip_stream_create()
    pm.check(lib.pmetal_hip_record_begin(stream))
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(lins), stream))
    rec = lib.pmetal_hip_record_end(stream)
    if not rec:
        raise RuntimeError(lib.pmetal_hip_last_error_message())
    timer.stream = stream
    ev_ms, wall_ms = timer.run(lambda: pm.check(lib.pmetal_hip_replay(rec, stream)), args.steps, args.warmup)
    timer.stream = None
    pm.check(lib.pmetal_hip_recording_destroy(rec))
    tok_s = args.steps / (ev_ms * 1e-3)
    gbs = total_bytes * tok_s / 1e9
    return {
        "value": tok_s, "ms_per_step": wall_ms / args.steps, "event_ms_per_step": ev_ms / args.steps,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_qgemv_q4k / k_qgemv_q6k (197 projections in 113 launches)" if model == "qwen3_0.6b"
                     else "k_qgemv_q4k_chunk / k_qgemv_q6k_chunk (225 projections)",
                     "bytes_per_step": total_bytes},
        "extra": {"launches_per_token": len(lins), "q6k_tensors": sum(1 for l in lins if l[3] == Q6K),
                  "submission": "one recorded sequence per token", "eager_tokens_per_s": round(args.steps / (eager_ms * 1e-3), 1)},
    }, (Q4K, 0, 0)


def bench_quantize(args):
    """f32 -> Q4_K_M over a random-init Llama-3-8B-shaped weight set resident in HBM (32 GB in, 5 GB out)."""
    pm, _lib, lib = load()
    timer = Timer(pm, lib)
    tensors = llama3_8b_tensors(pm)
    n_total = sum(n * k for _, n, k, _ in tensors)
    out_total = sum(lib.pmetal_hip_tensor_size(t, n * k) for _, n, k, t in tensors)
    src = pm.DeviceBuffer(4 * n_total)
    dst = pm.DeviceBuffer(out_total + 256 * len(tensors))
    jobs, so, do = [], 0, 0
    for i, (name, n, k, t) in enumerate(tensors):
        ne = n * k
        pm.check(lib.pmetal_hip_fill_normal_f32(src.ptr + 4 * so, ne, 7000 + i, 0.02, 1e-3, 0.5, None))
        nb = lib.pmetal_hip_tensor_size(t, ne)
        jobs.append((t, src.ptr + 4 * so, ne, dst.ptr + do, nb))
        so += ne
        do += (nb + 255) // 256 * 256
    pm.check(lib.pmetal_hip_sync(None))

    def one_by_one():
        for t, sp, ne, dp, nb in jobs:
            pm.check(lib.pmetal_hip_quantize_dev(t, sp, ne, dp, nb, None), "quantize")

    # the model's tensor loop as one call: the library spreads the independent tensors over two streams, so that one
    # kernel's last workgroups overlap the next kernel's first (same kernels, same bytes)
    descs = (_lib.QuantizeDesc * len(jobs))()
    for i, (t, sp, ne, dp, nb) in enumerate(jobs):
        descs[i] = _lib.QuantizeDesc(t, 0, sp, ne, dp, nb)

    def step():
        pm.check(lib.pmetal_hip_quantize_batch_dev(descs, len(jobs), None), "quantize batch")

    single_ms, _ = timer.run(one_by_one, max(args.steps // 4, 2), 1)
    single_ms /= max(args.steps // 4, 2)
    ev_ms, wall_ms = timer.run(step, args.steps, args.warmup)
    gbs_in = 4.0 * n_total * args.steps / (ev_ms * 1e-3) / 1e9
    gbs_total = (4.0 * n_total + out_total) * args.steps / (ev_ms * 1e-3) / 1e9
    q6 = sum(n * k for _, n, k, t in tensors if t == Q6K)
    return {
        "value": gbs_in, "ms_per_step": wall_ms / args.steps, "event_ms_per_step": ev_ms / args.steps,
        "roofline": {"bound": "hbm", "achieved": round(gbs_total, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs_total / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_quantize_q4k / k_quantize_q6k", "bytes_per_step": 4 * n_total + out_total},
        "extra": {"elements": n_total, "q6k_fraction": round(q6 / n_total, 4), "tensors": len(tensors),
                  "output_bytes": out_total, "entry_point": "pmetal_hip_quantize_batch_dev (one call per step)",
                  "one_call_per_tensor_ms": round(single_ms, 3), "one_call_per_tensor_GBs": round(4.0 * n_total / (single_ms * 1e-3) / 1e9, 1)},
    }, (Q4K, 0, 0)


WORKLOADS = {
    "gemv_q4k_14336x4096": dict(kind="gemv", n=14336, k=4096, metric="Q4_K GEMV GB/s @14336x4096", unit="GB/s",
                                dtype="bf16"),
    "gemv_q4k_4096x14336": dict(kind="gemv", n=4096, k=14336, metric="Q4_K GEMV GB/s @4096x14336", unit="GB/s",
                                dtype="bf16"),
}
WORKLOADS["gemv_q6k_14336x4096"] = dict(kind="gemv", n=14336, k=4096, type=Q6K, metric="Q6_K GEMV GB/s @14336x4096", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q3k_14336x4096"] = dict(kind="gemv", n=14336, k=4096, type=11, metric="Q3_K GEMV GB/s @14336x4096", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q2k_14336x4096"] = dict(kind="gemv", n=14336, k=4096, type=10, metric="Q2_K GEMV GB/s @14336x4096", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q5k_6144x4096"] = dict(kind="gemv", n=6144, k=4096, type=13, metric="Q5_K GEMV GB/s @6144x4096 (fused attn_qkv)", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q6k_18944x3584"] = dict(kind="gemv", n=18944, k=3584, type=Q6K, metric="Q6_K GEMV GB/s @18944x3584", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q6k_151936x1024"] = dict(kind="gemv", n=151936, k=1024, type=Q6K, metric="Q6_K GEMV GB/s @151936x1024 (output projection of a small model)", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q8_0_14336x4096"] = dict(kind="gemv", n=14336, k=4096, type=Q8_0, metric="Q8_0 GEMV GB/s @14336x4096", unit="GB/s", dtype="bf16")
WORKLOADS["gemv_q4k_q8k_14336x4096"] = dict(kind="gemv_q8k", n=14336, k=4096, type=Q4K, unit="GB/s", dtype="i8",
                                            metric="Q4_K x Q8_K integer-dot GEMV GB/s @14336x4096 (activation quantize included)")
WORKLOADS["gemv_q6k_q8k_14336x4096"] = dict(kind="gemv_q8k", n=14336, k=4096, type=Q6K, unit="GB/s", dtype="i8",
                                            metric="Q6_K x Q8_K integer-dot GEMV GB/s @14336x4096 (activation quantize included)")
WORKLOADS["calibrate_14336x4096"] = dict(kind="calibrate", n=14336, k=4096, unit="GB/s", dtype="f32",
                                         metric="KL calibration GB/s of f32 evaluated (6 candidates, quantize + dequantize + score) @14336x4096")
WORKLOADS["decode_qwen3_0.6b_q4km"] = dict(kind="decode", metric="Q4_K_M decode linears tokens/s (Qwen3-0.6B shape)", unit="tokens/s",
                                           dtype="bf16")
WORKLOADS["decode_llama3_8b_q4km"] = dict(kind="decode", model="llama3_8b", metric="Q4_K_M decode linears tokens/s (Llama-3-8B shape)",
                                          unit="tokens/s", dtype="bf16")
WORKLOADS["quantize_llama3_8b_q4km"] = dict(kind="quantize", metric="f32->Q4_K_M quantize GB/s of f32 consumed (Llama-3-8B shape)",
                                            unit="GB/s", dtype="f32")
WORKLOADS["dequantize_14336x4096"] = dict(kind="dequantize", n=14336, k=4096, unit="GB/s", dtype="f32",
                                          metric="Q4_K dequantize GB/s (blocks read + f32 written) @14336x4096")
for _m in (16, 64, 128, 512, 2048):
    WORKLOADS[f"gemm_q4k_m{_m}"] = dict(kind="gemm", m=_m, n=14336, k=4096, metric=f"Q4_K GEMM TFLOPS @M={_m},K=4096,N=14336",
                                        unit="TFLOP/s", dtype="f16", type=Q4K)
WORKLOADS["gemm_q6k_m512"] = dict(kind="gemm", m=512, n=14336, k=4096, metric="Q6_K GEMM TFLOPS @M=512,K=4096,N=14336",
                                  unit="TFLOP/s", dtype="f16", type=Q6K)
WORKLOADS["gemm_q8_0_m512"] = dict(kind="gemm", m=512, n=14336, k=4096, metric="Q8_0 GEMM TFLOPS @M=512,K=4096,N=14336",
                                   unit="TFLOP/s", dtype="f16", type=Q8_0)
WORKLOADS["gemm_q8_0_m16"] = dict(kind="gemm", m=16, n=14336, k=4096, metric="Q8_0 GEMM TFLOPS @M=16,K=4096,N=14336",
                                  unit="TFLOP/s", dtype="f16", type=Q8_0)
WORKLOADS["gemm_q6k_m16"] = dict(kind="gemm", m=16, n=14336, k=4096, metric="Q6_K GEMM TFLOPS @M=16,K=4096,N=14336",
                                 unit="TFLOP/s", dtype="f16", type=Q6K)
for _name, _t in (("q5k", 13), ("q3k", 11), ("q2k", 10)):
    WORKLOADS[f"gemm_{_name}_m16"] = dict(kind="gemm", m=16, n=14336, k=4096, unit="TFLOP/s", dtype="f16", type=_t,
                                          metric=f"{_name.upper().replace('K', '_K')} GEMM TFLOPS @M=16,K=4096,N=14336")
for _name, _t in (("q5k", 13), ("q3k", 11), ("q2k", 10)):  # (their own kernels; the form re-blocked into Q6_K is timed beside them)
    WORKLOADS[f"gemm_{_name}_m512"] = dict(kind="gemm", m=512, n=14336, k=4096, unit="TFLOP/s", dtype="f16", type=_t,
                                           metric=f"{_name.upper().replace('K', '_K')} GEMM TFLOPS (nominal flops) @M=512,K=4096,N=14336")


def set_recorded_traffic(roofline, workload):
    rec = RECORDED_TRAFFIC.get(workload)
    roofline["traffic"] = rec[0] if rec else None
    if rec:
        roofline["traffic_source"] = f"recorded constant from {rec[1]} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE), not measured in this run"


def other_parts(args):
    """The other parts of the metric and of its configurations: the Q4_K GEMM at M = 512 (with the sweep over M), the
    Llama-3-8B-shaped f32 -> Q4_K_M quantizer, the GEMV's second shape and the decode step of the small model."""
    import copy
    out = {}
    a = copy.copy(args)
    a.steps, a.warmup = max(args.steps, 50), max(args.warmup, 5)
    a.dense_library = True
    res, _ = bench_gemm(a, 512, 14336, 4096, Q4K)
    wl = WORKLOADS["gemm_q4k_m512"]
    set_recorded_traffic(res["roofline"], "gemm_q4k_m512")
    out["gemm_q4k_m512"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                            "steps": a.steps, "ms_per_step": round(res["ms_per_step"], 5), "roofline": res["roofline"],
                            "extra": res["extra"]}
    if not args.no_cpu_baseline:
        out["gemm_q4k_m512"]["cpu_baseline"] = cpu_baseline_gemm(Q4K, 512, 14336, 4096, budget_s=3.0)
    # the sweep of the prefill configuration: the crossover from the GEMV to the matrix cores
    a.dense_library = False
    for m in (16, 64, 128, 2048):
        a.steps, a.warmup = (50, 5) if m <= 128 else (20, 3)
        res, _ = bench_gemm(a, m, 14336, 4096, Q4K)
        wl = WORKLOADS[f"gemm_q4k_m{m}"]
        hbm = None
        if m <= 128:  # short batches are bound by reading the weights
            gb = (14336 * 16 * 144 + 2 * m * 4096 + 2 * m * 14336) / (res["roofline"]["us_per_launch"] * 1e-6) / 1e9
            hbm = {"bound": "hbm", "achieved": round(gb, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gb / HBM_PEAK_GBS, 4)}
        out[f"gemm_q4k_m{m}"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                                 "steps": a.steps, "us_per_call": res["roofline"]["us_per_launch"], "roofline": res["roofline"],
                                 **({"roofline_hbm": hbm} if hbm else {}), "weights": res["extra"]["weights"]}
    # the other block types of the recipe's files at the prefill shape (Q6_K: attn_v / ffn_down of half the layers and the
    # output matrix; Q5_K: a fused attn_qkv)
    for name, t in (("gemm_q6k_m512", Q6K), ("gemm_q5k_m512", 13)):
        a.steps, a.warmup = 30, 5
        res, _ = bench_gemm(a, 512, 14336, 4096, t)
        wl = WORKLOADS[name]
        out[name] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                     "steps": a.steps, "us_per_call": res["roofline"]["us_per_launch"], "roofline": res["roofline"],
                     "two_weights_sharing_x_us_per_weight": res["extra"]["two_weights_sharing_x_us_per_weight"]}
    # the second shape of the decode configuration (the down projection)
    a = copy.copy(args)
    a.steps, a.warmup = max(args.steps // 4, 10), max(args.warmup // 4, 2)
    res, _ = bench_gemv(a, 4096, 14336, Q4K)
    wl = WORKLOADS["gemv_q4k_4096x14336"]
    set_recorded_traffic(res["roofline"], "gemv_q4k_4096x14336")
    out["gemv_q4k_4096x14336"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                                  "steps": a.steps, "ms_per_step": round(res["ms_per_step"], 5), "roofline": res["roofline"],
                                  "extra": res["extra"]}
    # the decode step of the small model (tokens/s over its linear projections)
    a = copy.copy(args)
    a.steps, a.warmup = max(args.steps, 100), max(args.warmup, 10)
    res, _ = bench_decode(a, "qwen3_0.6b")
    wl = WORKLOADS["decode_qwen3_0.6b_q4km"]
    out["decode_qwen3_0.6b_q4km"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                                     "steps": a.steps, "ms_per_step": round(res["ms_per_step"], 5), "roofline": res["roofline"],
                                     "extra": res["extra"]}
    # ... and of an 8B-class model, whose projections are long enough to stream (informative: not one of the configurations)
    a = copy.copy(args)
    a.steps, a.warmup = 20, 3
    res, _ = bench_decode(a, "llama3_8b")
    wl = WORKLOADS["decode_llama3_8b_q4km"]
    out["decode_llama3_8b_q4km"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "dtype": wl["dtype"],
                                    "steps": a.steps, "ms_per_step": round(res["ms_per_step"], 5), "roofline": res["roofline"]}
    a = copy.copy(args)
    a.steps, a.warmup = 5, 1
    res, _ = bench_quantize(a)
    wl = WORKLOADS["quantize_llama3_8b_q4km"]
    set_recorded_traffic(res["roofline"], "quantize_llama3_8b_q4km")
    out["quantize_llama3_8b_q4km"] = {"metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"],
                                      "dtype": wl["dtype"], "steps": a.steps, "ms_per_step": round(res["ms_per_step"], 5),
                                      "roofline": res["roofline"], "extra": res["extra"]}
    if not args.no_cpu_baseline:
        out["quantize_llama3_8b_q4km"]["cpu_baseline"] = cpu_baseline_quantize(budget_s=3.0)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gemv_q4k_14336x4096", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-workloads", action="store_true",
                    help="default workload only: do not also time the GEMM and quantizer parts of the metric")
    ap.add_argument("--dense-library", action="store_true",
                    help="GEMM workloads: also time torch.matmul (f16, same shape) as a yardstick; the default run does so for M = 512")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain streaming kernel of known size (f32 -> bf16 over 2^24 elements: 64 MiB read, "
                         "32 MiB written) so that profiler byte counters can be scaled against it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)")
    wl = WORKLOADS[args.workload]
    if wl["kind"] == "gemm":
        res, (t, n, k) = bench_gemm(args, wl["m"], wl["n"], wl["k"], wl["type"])
    elif wl["kind"] == "decode":
        res, (t, n, k) = bench_decode(args, wl.get("model", "qwen3_0.6b"))
    elif wl["kind"] == "quantize":
        res, (t, n, k) = bench_quantize(args)
    elif wl["kind"] == "dequantize":
        res, (t, n, k) = bench_dequantize(args, wl["n"], wl["k"])
    elif wl["kind"] == "gemv_q8k":
        res, (t, n, k) = bench_gemv_q8k(args, wl["n"], wl["k"], wl["type"])
    elif wl["kind"] == "calibrate":
        res, (t, n, k) = bench_calibrate(args, wl["n"], wl["k"])
    else:
        res, (t, n, k) = bench_gemv(args, wl["n"], wl["k"], wl.get("type", Q4K))
    out = {
        "metric": wl["metric"], "value": round(res["value"], 1), "unit": wl["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(res["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": wl["dtype"],
        "data": ("synthetic: N(0,0.02) f32 with 0.1% outliers at +-0.5, generated on the device" if wl["kind"] == "quantize"
                 else "synthetic: N(0,0.02) f32 weights generated and quantized on the device, x ~ N(0,1) f32" if wl["kind"] == "gemv_q8k"
                 else "synthetic: N(0,0.02) f32 with 0.1% outliers at +-0.5, generated on the device" if wl["kind"] == "calibrate"
                 else "synthetic: N(0,0.02) f32 weights generated and quantized on the device, x ~ N(0,1) bf16"),
        "config": {"workload": args.workload, "element_order": "GGML" if wl["kind"] == "calibrate" else "REF",
                   "step": {"gemm": "one GEMM launch (activation pre-pass + MFMA kernel)",
                            "gemv": "8 sweeps of 16 back-to-back GEMV launches, one per distinct weight tensor (HBM-resident: 528 MB for Q4_K), replayed from a recorded launch sequence",
                            "gemv_q8k": "16 x (activations f32 -> Q8_K, integer-dot GEMV) over 16 distinct weight tensors",
                            "calibrate": "one tensor resident in HBM: 6 candidates x (quantize, fused dequantize-and-score, f64 score read back)",
                            "decode": "all batch-1 projections of one token (197 for Qwen3-0.6B, 225 for Llama-3-8B), back to back on one stream",
                            "dequantize": "two tensors of 14336 x 4096, blocks resident in HBM",
                            "quantize": "all 226 tensors of the model, f32 resident in HBM, one pmetal_hip_quantize_batch_dev call"}[wl["kind"]]},
        "roofline": res["roofline"], "extra": res["extra"],
    }
    out["extra"]["event_ms_per_step"] = round(res["event_ms_per_step"], 5)
    if wl["kind"] == "gemv":
        # `dtype` names the activation type handed over; the kernels of these (large) shapes multiply in integers
        if "_q4k_" in args.workload:
            out["config"]["arithmetic"] = ("bf16 activations converted to 20-bit fixed point per 32-element block, five 4-bit digit planes, "
                                           "v_dot8_u32_u4 against the packed nibbles, f32 block scales and accumulation")
        else:
            out["config"]["arithmetic"] = ("bf16 activations converted exactly to fixed-point int8 digit planes, v_dot4_i32_i8 against "
                                           "the quantized weights, f32 block scales and accumulation")
    set_recorded_traffic(out["roofline"], args.workload)
    if args.calibrate:
        pm, _lib, lib = load()
        n_cal = 1 << 24
        src, dst = pm.DeviceBuffer(4 * n_cal), pm.DeviceBuffer(2 * n_cal)
        pm.check(lib.pmetal_hip_fill_normal_f32(src.ptr, n_cal, 1, 1.0, 0.0, 0.0, None))
        for _ in range(5):
            pm.check(lib.pmetal_hip_f32_to_bf16_dev(src.ptr, dst.ptr, n_cal, None))
        pm.check(lib.pmetal_hip_sync(None))
    if args.workload == "gemv_q4k_14336x4096" and not args.no_extra_workloads:
        # the other two parts of the headline metric ("Q4_K GEMM TFLOPS; quantize GB/s"), timed in the same run
        out["extra"]["other_parts_of_the_metric"] = other_parts(args)
    if not args.no_cpu_baseline:
        if wl["kind"] == "gemv":
            out["cpu_baseline"] = cpu_baseline_gemv(t, n, k)
        elif wl["kind"] == "gemv_q8k":
            out["cpu_baseline"] = cpu_baseline_gemv_q8k(t, n, k)
        elif wl["kind"] == "calibrate":
            out["cpu_baseline"] = cpu_baseline_calibrate()
        elif wl["kind"] == "quantize":
            out["cpu_baseline"] = cpu_baseline_quantize()
        elif wl["kind"] == "gemm":
            out["cpu_baseline"] = cpu_baseline_gemm(wl["type"], wl["m"], wl["n"], wl["k"])
        elif wl["kind"] == "dequantize":
            out["cpu_baseline"] = cpu_baseline_dequantize()
        else:
            out["cpu_baseline"] = cpu_baseline_decode(load()[0], wl.get("model", "qwen3_0.6b"))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
