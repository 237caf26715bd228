#!/usr/bin/env python3
"""Benchmark of the packed-low-precision hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

A "step" is one E4M3-packed GEMV of the 16384 x 16384 workload (FP32 accumulate) with the
operands already resident in HBM.  Four distinct packed matrices (1 GiB in total) are
rotated so that neither L2 nor the 256 MB Infinity Cache can serve the stream.  The single
JSON line printed at the end carries the headline value (microseconds per GEMV), the
roofline record of the GEMV kernel -- with the matrix-core record of the metric's second half,
flash attention d = 64 L = 8192, nested in it -- and the CPU baseline (torch-CPU restatement of
the reference's pack + decode + fp32 compute, timed on the host cores of this box, one leg per
configuration); `extra` holds the other workloads (the reference harness's GEMV grid in both
modes, dot, pack / unpack, flash attention vs fp16 SDPA, paged decode, the decode step) with a
roofline record each (`extra.roofline` HBM bound, `extra.roofline_mfma` matrix-core bound);
every record says how it was timed ("events": back-to-back calls between HIP events; "graph":
replay of captured calls, for kernels shorter than the host's per-call cost).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_F16_TFLOPS = 2500.0  # dense fp16/bf16, published
MFMA_PEAK_F8_TFLOPS = 5000.0   # dense fp8/bf8, published
WARM_MS = 40.0                  # warm-up time of the attention series (ours and SDPA alike)


def gpu_time_us(fn, steps, warmup, sync, warm_ms=0.0, gate=3):
    """Average microseconds per call over `steps` back-to-back calls (HIP events on the
    stream the kernels are launched on: torch's current stream).  With `warm_ms` the warm-up calls are
    repeated until that many milliseconds of back-to-back work have passed: the first tens of
    milliseconds of a series run below the sustained clock.  `gate` untimed calls right after the last
    synchronize keep the device busy while the host enqueues the start event and the first timed calls
    (otherwise the host's per-call cost before the first launch is counted as kernel time)."""
    import torch
    t0 = time.perf_counter()
    for i in range(warmup):
        fn(i)
    sync()
    while (time.perf_counter() - t0) * 1000.0 < warm_ms:
        for i in range(max(warmup, 1)):
            fn(i)
        sync()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(gate):
        fn(i)
    start.record()
    for i in range(steps):
        fn(gate + i)
    stop.record()
    sync()
    return start.elapsed_time(stop) * 1000.0 / steps


def gpu_time_graph_us(fn, calls, sync, replays=10):
    """Device microseconds per call for kernels shorter than the host's per-call cost (the Python wrapper:
    output allocation, stream lookup, ctypes call, ~8 us): `calls` invocations are captured in one HIP graph
    and the graph is replayed back to back."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(calls):
            fn(i)                                             # warm-up outside the capture (allocations, module load)
    torch.cuda.current_stream().wait_stream(side)
    sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(calls):
            fn(i)
    for _ in range(3):
        graph.replay()
    sync()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    sync()
    return start.elapsed_time(stop) * 1000.0 / (replays * calls)


def gpu_time_auto_us(fn, calls, steps, warmup, sync, warm_ms=0.0):
    """(microseconds per call, timing method).  Back-to-back calls between HIP events ("events") unless a call
    is shorter than the host's per-call cost (~12 us of wrapper and dispatch): then the device time alone, from
    the replay of `calls` captured invocations ("graph").  One method per figure, never the smaller of two."""
    us = gpu_time_us(fn, steps, warmup, sync, warm_ms)
    if us >= 12.0:
        return us, "events"
    return gpu_time_graph_us(fn, calls, sync), "graph"


def _source_hash(rel_paths) -> str:
    """sha256 (first 16 hex digits) over the kernel sources a counter figure belongs to."""
    import hashlib
    h = hashlib.sha256()
    for rel in rel_paths:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def load_traffic() -> dict:
    """HBM bytes per launch from the committed rocprofv3 counter summary: lines
    `hbm_bytes_per_launch <key> <bytes> <sha> <source>[,<source>...]`.  A figure whose kernel sources
    have changed since the counters were taken is reported as stale (traffic = null) instead of being
    carried along silently."""
    out = {}
    path = os.path.join(ROOT, "profiles", "bench_hbm_traffic.md")
    if not os.path.exists(path):
        return out
    for ln in open(path):
        f = ln.split()
        if len(f) == 5 and f[0] == "hbm_bytes_per_launch":
            try:
                fresh = _source_hash(f[4].split(",")) == f[3]
            except OSError:
                fresh = False
            out[f[1]] = (int(f[2]), fresh)
    return out


def load_mfma_busy() -> dict:
    """Matrix-core busy fraction per attention workload from the committed rocprofv3 counter summary: lines
    `mfma_busy <key> <SQ_VALU_MFMA_BUSY_CYCLES / SQ_BUSY_CYCLES per SIMD> <sha> <source>[,<source>...]`; stale figures
    (kernel source changed since) are reported as null."""
    out = {}
    path = os.path.join(ROOT, "profiles", "bench_sq_counters.md")
    if not os.path.exists(path):
        return out
    for ln in open(path):
        f = ln.split()
        if len(f) == 5 and f[0] == "mfma_busy":
            try:
                fresh = _source_hash(f[4].split(",")) == f[3]
            except OSError:
                fresh = False
            out[f[1]] = (float(f[2]), fresh)
    return out


def roofline_record(traffic_table, key, kernel, algorithmic_bytes, us, launches_per_call=1, timing="events", note=None):
    """`roofline`-style record of an HBM-bound workload: achieved = algorithmic bytes / measured time."""
    achieved = algorithmic_bytes / (us * 1e-6) / 1e9
    t = traffic_table.get(key)
    rec = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": t[0] if t and t[1] else None, "kernel": kernel,
           "algorithmic_bytes": int(algorithmic_bytes), "us": round(us, 3), "timing": timing}
    if t and not t[1]:
        rec["traffic_note"] = "stale: the kernel source changed since the counters in profiles/bench_hbm_traffic.md were taken"
    if launches_per_call != 1:
        rec["launches_per_call"] = launches_per_call
    if note:
        rec["note"] = note
    return rec


def mfma_record(busy_table, key, kernel, flops, us, fp8_share, sdpa_us=None):
    """`roofline`-style record of a matrix-core-bound workload.  `peak` is the dense fp16 MFMA peak; when a share of
    the flops runs at the FP8 rate (the E5M2 score product on the bf8 matrix instructions) `peak_blended` is the rate
    at which the same flop mix would run with every matrix instruction at its own peak, and both fractions are given."""
    achieved = flops / (us * 1e-6) / 1e12
    blended = 1.0 / (fp8_share / MFMA_PEAK_F8_TFLOPS + (1.0 - fp8_share) / MFMA_PEAK_F16_TFLOPS)
    b = busy_table.get(key)
    rec = {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_PEAK_F16_TFLOPS, "unit": "TFLOP/s",
           "frac": round(achieved / MFMA_PEAK_F16_TFLOPS, 4), "peak_blended": round(blended, 1),
           "frac_blended": round(achieved / blended, 4), "fp8_rate_flop_share": fp8_share, "traffic": None,
           "kernel": kernel, "flops": int(flops), "us": round(us, 1), "timing": "events",
           "mfma_busy": b[0] if b and b[1] else None}
    if b and not b[1]:
        rec["mfma_busy_note"] = "stale: the kernel source changed since the counters in profiles/bench_sq_counters.md were taken"
    if sdpa_us is not None:
        rec["sdpa_fp16_same_gpu_us"] = round(sdpa_us, 1)
        rec["speedup_vs_sdpa_fp16"] = round(sdpa_us / us, 3)
    return rec


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extra", action="store_true", help="only the headline GEMV workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--prewarm", type=int, default=1200,
                    help="untimed launches of the headline kernel that bring the clocks up before the warm-up steps "
                         "(counter runs under rocprofv3 --pmc use a small number: counters do not depend on the clock)")
    ap.add_argument("--warm-ms", type=float, default=WARM_MS,
                    help="milliseconds of back-to-back warm-up calls before each attention / decode series")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (known traffic) to scale rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    warm_ms = args.warm_ms
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (every routine is single-device); --gpus must be 1",
              file=sys.stderr)
        return 2

    import torch

    import feather_amd as feather
    from feather_amd import _native as N

    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    dev = torch.device("cuda:0")
    sync = torch.cuda.synchronize
    N.lib()
    g = torch.Generator(device=dev).manual_seed(2)   # synthetic inputs are drawn on the device

    def randn(*shape):
        return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32)

    # ---------------------------------------------------------------- headline: E4M3 GEMV 16384^2
    M = K = 16384
    NBUF = 4

    def make_matrix(mode):
        x = randn(M, K)
        x = torch.where(torch.rand(M, K, generator=g, device=dev) < 0.01, x * 1e-3, x)  # zero-exponent E4M3 codes
        return feather.pack_fp8_tensor(x.half(), mode=mode)

    mats = {"E4M3": [make_matrix("E4M3") for _ in range(NBUF)]}
    v16 = randn(K).half()
    vecs = {m: feather.pack_fp8_tensor(v16, mode=m) for m in ("E4M3", "E5M2")}
    gemv_bytes = M * K + K + 4 * M                             # 1 B per code, vector once, fp32 out

    def gemv_step(mode):
        bufs, vp = mats[mode], vecs[mode]
        return lambda i: feather.gemv(bufs[i % NBUF], vp, original_shape=(M, K), mode=mode)

    # Clock ramp: the first tens of milliseconds of GPU work in a process run below the sustained clock
    # (three back-to-back series of 200 launches measured 45.7, 43.9 and 43.0 us), so the same launches
    # run for ~50 ms before the W warm-up steps; the timed region stays exactly K steps.
    PREWARM = args.prewarm
    sync()
    cold_us = gpu_time_us(gemv_step("E4M3"), args.steps, 0, sync, gate=0)   # the first series of the process, no warm-up at all
    for i in range(PREWARM):
        gemv_step("E4M3")(i)
    # the whole timed region, bracketed by synchronize on both sides
    for i in range(args.warmup):
        gemv_step("E4M3")(i)
    sync()
    # After a synchronize the queue is empty: the first launch reaches the device only after the host's
    # per-call cost (~15 us of wrapper and dispatch), which HIP events around K launches would count as
    # kernel time (0.7 us per launch at K = 20).  GATE untimed launches of the same kernel keep the device
    # busy while the host enqueues the start event and the first timed launches, so the events enclose
    # exactly K back-to-back launches; the wall clock covers all GATE + K launches.
    GATE = 3
    t0 = time.perf_counter()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    step = gemv_step("E4M3")
    for i in range(GATE):
        step(args.warmup + i)
    ev0.record()
    for i in range(args.steps):
        step(args.warmup + GATE + i)
    ev1.record()
    sync()
    wall_ms = (time.perf_counter() - t0) * 1000.0
    kern_us = ev0.elapsed_time(ev1) * 1000.0 / args.steps
    ms_per_step = wall_ms / (args.steps + GATE)

    if args.calibrate_copy:
        src = torch.empty(M * K // 4, dtype=torch.int32, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)                                      # reads 256 MiB, writes 256 MiB
        sync()
        del src, dst

    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/bench_hbm_traffic.md)
    ttab = load_traffic()
    headline = roofline_record(ttab, "gemv_e4m3_16384", "gemv_fp8_kernel<E4M3>", gemv_bytes, kern_us)

    extra = {"gemv_e4m3_16384_cold_first_series_us": round(cold_us, 2)}   # same kernel, first series: no warm-up, first-launch cost included
    rl = {}                                                               # roofline records of the other HBM-bound workloads
    arl = {}                                                              # roofline records of the matrix-core-bound workloads (attention)
    if not args.no_extra:
        # cache-resident figure (one matrix re-used): reported separately, never the headline
        one = mats["E4M3"][0]
        extra["gemv_e4m3_16384_same_buffer_us"] = round(
            gpu_time_us(lambda i: feather.gemv(one, vecs["E4M3"], original_shape=(M, K), mode="E4M3"), 100, 10, sync), 2)
        # the reference harness's GEMV grid (benchmark/bench_gemv.py:14-15 and README.md:33-35: 4096^2, 8192^2,
        # 16384 x 8192, 16384^2) in E4M3 first, on views into the four rotating 256 MiB buffers (>= 4 distinct operands
        # of every shape, 1 GiB cycled), then the same in E5M2
        from feather_amd.routines.gemv import gemv_fp8_batched_acc_fp32_gpu

        def gemv_grid(mode):
            bufs = mats[mode]
            for Ms in (4096, 8192, 16384):
                for Ks in (4096, 8192, 16384):
                    if Ms == M and Ks == K:
                        continue                                 # 16384^2 is the headline (E4M3) / its own series (E5M2)
                    words = Ms * Ks // 4
                    per = (M * K // 4) // words
                    views = [b[i * words:(i + 1) * words] for b in bufs for i in range(per)]
                    vp = feather.pack_fp8_tensor(v16[:Ks], mode=mode)
                    call = lambda i: feather.gemv(views[i % len(views)], vp, original_shape=(Ms, Ks), mode=mode)
                    us, how = gpu_time_auto_us(call, min(64, len(views)), args.steps, args.warmup, sync, 10.0)
                    key = f"gemv_{mode.lower()}_{Ms}x{Ks}" if Ms != Ks else f"gemv_{mode.lower()}_{Ms}"
                    extra[key + "_us"] = round(us, 2)
                    extra[key + "_GBps"] = round((Ms * Ks + Ks + 4 * Ms) / us / 1e3, 1)
                    rl[key] = roofline_record(ttab, key, f"gemv_fp8_kernel<{mode}>", Ms * Ks + Ks + 4 * Ms, us, timing=how)
            # batched GEMV: the rotating matrices against 32 vectors (weights streamed once per batch)
            xb = feather.pack_fp8_tensor(randn(32, K).half(), mode=mode)
            us = gpu_time_us(lambda i: gemv_fp8_batched_acc_fp32_gpu(bufs[i % NBUF], xb, (M, K), 32, mode), 50, 10, sync)
            key = f"gemv_batched_{mode.lower()}_16384_x32"
            extra[key + "_us"] = round(us, 2)
            extra[key + "_GBps"] = round((M * K + 32 * K + 4 * 32 * M) / us / 1e3, 1)
            rl[key] = roofline_record(ttab, key, f"gemv_batched_kernel<{mode}>", M * K + 32 * K + 4 * 32 * M, us)

        gemv_grid("E4M3")
        del mats["E4M3"]
        torch.cuda.empty_cache()
        mats["E5M2"] = [make_matrix("E5M2") for _ in range(NBUF)]
        us = gpu_time_us(gemv_step("E5M2"), args.steps, PREWARM + args.warmup, sync)   # same clock pre-warm as the headline
        extra["gemv_e5m2_16384_us"] = round(us, 2)
        extra["gemv_e5m2_16384_GBps"] = round(gemv_bytes / us / 1e3, 1)
        extra["gemv_e5m2_16384_hbm_frac"] = round(gemv_bytes / us / 1e3 / HBM_PEAK_GBS, 4)
        rl["gemv_e5m2_16384"] = roofline_record(ttab, "gemv_e5m2_16384", "gemv_fp8_kernel<E5M2>", gemv_bytes, us)
        gemv_grid("E5M2")
        # dot, n = 2^24: rotate through the big buffers (64 distinct operands of 16 MiB)
        from feather_amd.routines.dot import dot_fp16_acc_fp32_gpu
        n = 1 << 24
        xs = [b[i * (n // 4):(i + 1) * (n // 4)] for b in mats["E5M2"] for i in range(16)]
        for mode in ("E4M3", "E5M2"):
            us_call = gpu_time_us(lambda i: feather.dot(xs[(2 * i) % 64], xs[(2 * i + 1) % 64], mode=mode), args.steps,
                                  args.warmup, sync)
            extra[f"dot_{mode.lower()}_2p24_per_python_call_us"] = round(us_call, 2)   # host-bound: wrapper + two launches
            us = gpu_time_graph_us(lambda i: feather.dot(xs[(2 * i) % 64], xs[(2 * i + 1) % 64], mode=mode), 32, sync)
            extra[f"dot_{mode.lower()}_2p24_us"] = round(us, 2)
            extra[f"dot_{mode.lower()}_2p24_GBps"] = round((2 * n + 4) / us / 1e3, 1)
            rl[f"dot_{mode.lower()}_2p24"] = roofline_record(ttab, f"dot_{mode.lower()}_2p24", f"dot_kernel<{mode}> + dot_finish_kernel",
                                                              2 * n + 4, us, launches_per_call=2, timing="graph")
        # FP16-packed dot (reference dot_fp16_acc_fp32_gpu, benchmark/bench_dot.py:138-160), n = 2^24 elements: 2 B per
        # element and operand, operands of 32 MiB taken from the same rotating buffers
        xh = [b[i * (n // 2):(i + 1) * (n // 2)] for b in mats["E5M2"] for i in range(8)]
        us = gpu_time_graph_us(lambda i: dot_fp16_acc_fp32_gpu(xh[(2 * i) % 32], xh[(2 * i + 1) % 32]), 32, sync)
        extra["dot_fp16_2p24_us"] = round(us, 2)
        extra["dot_fp16_2p24_GBps"] = round((4 * n + 4) / us / 1e3, 1)
        rl["dot_fp16_2p24"] = roofline_record(ttab, "dot_fp16_2p24", "dot_kernel<FP16> + dot_finish_kernel", 4 * n + 4, us,
                                              launches_per_call=2, timing="graph")
        # the largest size of the reference harness (benchmark/bench_dot.py:15), n = 1 500 000
        nh = 1_500_000
        for kind, words, call in (("e5m2", nh // 4, lambda a, b: feather.dot(a, b, mode="E5M2")),
                                  ("fp16", nh // 2, lambda a, b: dot_fp16_acc_fp32_gpu(a, b))):
            ops = [mats["E5M2"][0][i * words:(i + 1) * words] for i in range(32)]
            us = gpu_time_graph_us(lambda i: call(ops[(2 * i) % 32], ops[(2 * i + 1) % 32]), 32, sync)
            extra[f"dot_{kind}_1500000_us"] = round(us, 2)
        # dot, n = 16384 (one workgroup, one launch: latency bound)
        xs_s = [x[:4096] for x in xs]
        for mode in ("E4M3", "E5M2"):
            us = gpu_time_graph_us(lambda i: feather.dot(xs_s[(2 * i) % 64], xs_s[(2 * i + 1) % 64], mode=mode), 32, sync)
            extra[f"dot_{mode.lower()}_16384_us"] = round(us, 2)
        extra["dot_timing"] = "graph replay of 32 captured calls (device time; a Python call costs 8-11 us on the host)"
        del xh
        # pack throughput (2 B in + 1 B out per element)
        src = randn(8192, 16384).half()
        for mode in ("E5M2", "E4M3"):
            us = gpu_time_us(lambda i: feather.pack_fp8_tensor(src, mode=mode), 20, 3, sync)
            extra[f"pack_{mode.lower()}_134M_GBps"] = round(3 * src.numel() / us / 1e3, 1)
            rl[f"pack_{mode.lower()}_134M"] = roofline_record(ttab, f"pack_{mode.lower()}_134M", f"pack_fp8_kernel<{mode}>", 3 * src.numel(), us)
        # unpack (1 B in, 4 B fp32 out per element), ReLU on packed E5M2, fp16 container (2 B in + 2 B out)
        from feather_amd.routines.activations import relu1d_fp8_ret_fp32_feather_gpu
        words = mats["E5M2"][0][: src.numel() // 4]
        for mode, sem in (("E4M3", "ieee"), ("E4M3", "kernel"), ("E5M2", "ieee")):
            us = gpu_time_us(lambda i: feather.unpack_fp8_tensor(words, mode=mode, semantics=sem), 20, 3, sync)
            extra[f"unpack_{mode.lower()}_{sem}_f32_134M_GBps"] = round(5 * src.numel() / us / 1e3, 1)
            rl[f"unpack_{mode.lower()}_{sem}_134M"] = roofline_record(ttab, f"unpack_{mode.lower()}_{sem}_134M",
                                                                       f"unpack_fp8_kernel<{mode}, {sem}>", 5 * src.numel(), us)
        us = gpu_time_us(lambda i: relu1d_fp8_ret_fp32_feather_gpu(words, src.numel()), 20, 3, sync)
        extra["relu_e5m2_f32_134M_GBps"] = round(5 * src.numel() / us / 1e3, 1)
        us = gpu_time_us(lambda i: feather.pack_fp16_tensor(src), 20, 3, sync)
        extra["pack_fp16_134M_GBps"] = round(4 * src.numel() / us / 1e3, 1)
        del src, words
        del mats["E5M2"], xs
        torch.cuda.empty_cache()
        # flash attention, B4 H16 d64, E5M2, vs fp16 SDPA on the same GPU (both sides get WARM_MS of
        # back-to-back warm-up calls: the first tens of milliseconds of a series run below the sustained clock)
        busy = load_mfma_busy()
        for L in (4096, 8192):
            B, H, d = 4, 16, 64
            qkv16 = [randn(B, H, L, d).half() for _ in range(3)]
            pk = [feather.pack_fp8_tensor(t, mode="E5M2").view(B, H, L, d // 4) for t in qkv16]
            us = gpu_time_us(lambda i: feather.flash_attention_fp8_e5m2_acc_fp32_gpu(pk[0], pk[1], pk[2], L, d // 4),
                             10, 10, sync, warm_ms)
            flops = 4.0 * B * H * L * L * d
            us_sdpa = gpu_time_us(lambda i: torch.nn.functional.scaled_dot_product_attention(*qkv16), 10, 10, sync, warm_ms)
            key = f"flash_attn_e5m2_b4h16_d64_L{L}"
            extra[key + "_us"] = round(us, 1)
            extra[key + "_TFLOPs"] = round(flops / us / 1e6, 1)
            extra[key + "_mfma_frac"] = round(flops / us / 1e6 / MFMA_PEAK_F16_TFLOPS, 4)
            extra[f"sdpa_fp16_b4h16_d64_L{L}_us"] = round(us_sdpa, 1)
            # Q K^T (half the flops) runs on the bf8 matrix instruction at the FP8 rate, P V on the fp16 one
            arl[key] = mfma_record(busy, key, "flash_attn64_wide_kernel<E5M2>", flops, us, 0.5, us_sdpa)
            if L == 8192:   # causal prefill (half the flops) vs causal fp16 SDPA
                us = gpu_time_us(lambda i: feather.flash_attention_fp8_acc_fp32_gpu(pk[0], pk[1], pk[2], L, d // 4,
                                                                                    mode="E5M2", causal=True), 10, 10, sync, warm_ms)
                us_sdpa = gpu_time_us(lambda i: torch.nn.functional.scaled_dot_product_attention(*qkv16, is_causal=True),
                                      10, 10, sync, warm_ms)
                key = f"flash_attn_causal_e5m2_b4h16_d64_L{L}"
                extra[key + "_us"] = round(us, 1)
                extra[key + "_TFLOPs"] = round(flops / 2 / us / 1e6, 1)
                extra[f"sdpa_causal_fp16_b4h16_d64_L{L}_us"] = round(us_sdpa, 1)
                arl[key] = mfma_record(busy, key, "flash_attn64_wide_kernel<E5M2, causal>", flops / 2, us, 0.5, us_sdpa)
            if L == 8192:   # the same shape with E4M3 codes (fp16 score product: the E4M3 kernel decode is not the matrix core's format)
                pk4 = [feather.pack_fp8_tensor(t, mode="E4M3").view(B, H, L, d // 4) for t in qkv16]
                us = gpu_time_us(lambda i: feather.flash_attention_fp8_acc_fp32_gpu(pk4[0], pk4[1], pk4[2], L, d // 4, mode="E4M3"),
                                 10, 10, sync, warm_ms)
                key = f"flash_attn_e4m3_b4h16_d64_L{L}"
                extra[key + "_us"] = round(us, 1)
                extra[key + "_TFLOPs"] = round(flops / us / 1e6, 1)
                us_sdpa = extra[f"sdpa_fp16_b4h16_d64_L{L}_us"]
                arl[key] = mfma_record(busy, key, "flash_attn64_wide_kernel<E4M3>", flops, us, 0.0, us_sdpa)
                del pk4
            del qkv16, pk
        # wide heads: B1 H8, d = 256 / 512, E4M3, vs fp16 SDPA
        for d, L in ((256, 1024), (256, 4096), (256, 8192), (512, 1024), (512, 4096), (512, 8192)):
            B, H = 1, 8
            qkv16 = [randn(B, H, L, d).half() for _ in range(3)]
            pk = [feather.pack_fp8_tensor(t, mode="E4M3").view(B, H, L, d // 4) for t in qkv16]
            us = gpu_time_us(lambda i: feather.flash_attention_fp8_acc_fp32_gpu(pk[0], pk[1], pk[2], L, d // 4,
                                                                                mode="E4M3"), 10, 10, sync, warm_ms)
            key = f"flash_attn_e4m3_b1h8_d{d}_L{L}"
            extra[key + "_us"] = round(us, 1)
            extra[key + "_TFLOPs"] = round(4.0 * B * H * L * L * d / us / 1e6, 1)
            us_sdpa = gpu_time_us(lambda i: torch.nn.functional.scaled_dot_product_attention(*qkv16), 10, 10, sync, warm_ms)
            extra[f"sdpa_fp16_b1h8_d{d}_L{L}_us"] = round(us_sdpa, 1)
            arl[key] = mfma_record(busy, key, f"flash_attn_kernel<{d}, E4M3>", 4.0 * B * H * L * L * d, us, 0.0, us_sdpa)
            ws_bytes = int(N.lib().feather_flash_attn_workspace_bytes(B * H, L, d))
            if ws_bytes:   # a grid below 256 workgroups: key ranges over workgroups + a merge kernel (the wrapper's default)
                arl[key]["key_ranges"] = ws_bytes // (B * H * L * (d + 2) * 4)
                arl[key]["workspace_bytes"] = ws_bytes
            del qkv16, pk
        # the reference harness's own grid (benchmark/bench_attention.py:13-14): ONE head of 128 .. 8192 rows at head
        # dims 64 / 256 / 512, E5M2, the reference-named entry point with its tail semantics.  A single head makes 2 to
        # 128 workgroups; the wrapper hands the library a workspace and the key loop is cut into ranges over more
        # workgroups.  Device time by graph replay for both sides (the short ones are below the host's per-call cost).
        for d in (64, 256, 512):
            for L in (128, 256, 512, 1024, 4096, 8192):
                qkv16 = [randn(1, 1, L, d).half() for _ in range(3)]
                pk = [feather.pack_fp8_tensor(t[0, 0], mode="E5M2").view(L, d // 4) for t in qkv16]
                us = gpu_time_graph_us(lambda i: feather.flash_attention_fp8_e5m2_acc_fp32_gpu(pk[0], pk[1], pk[2], L, d // 4),
                                       16, sync)
                us_sdpa = gpu_time_graph_us(lambda i: torch.nn.functional.scaled_dot_product_attention(*qkv16), 16, sync)
                key = f"flash_attn_e5m2_h1_d{d}_L{L}"
                extra[key + "_us"] = round(us, 2)
                extra[f"sdpa_fp16_h1_d{d}_L{L}_us"] = round(us_sdpa, 2)
                kern = "flash_attn64_wide_kernel<E5M2>" if d == 64 else f"flash_attn_kernel<{d}, E5M2>"
                arl[key] = mfma_record(busy, key, kern, 4.0 * L * L * d, us, 0.5, us_sdpa)
                arl[key]["timing"] = "graph"
                ws_bytes = int(N.lib().feather_flash_attn_workspace_bytes(1, L, d))
                arl[key]["key_ranges"] = ws_bytes // (L * (d + 2) * 4) if ws_bytes else 1
                del qkv16, pk
        torch.cuda.empty_cache()
        # paged-attention decode, 32 sequences x 32 query heads over 4 KV heads, d=64, E4M3, blocks of 16
        # tokens scattered by a random block table; bytes = K and V codes of every context token once
        from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
        n_seq, Hq, Hkv, d, bs, cmax = 32, 32, 4, 64, 16, 4096
        nblk = n_seq * cmax // bs
        NKV = 4                                                  # K/V cache pairs rotated: 4 x 67 MB > the 256 MB Infinity Cache
        caches = [tuple(feather.pack_fp8_tensor(randn(nblk * Hkv * bs * d).half(), mode="E4M3").view(nblk, Hkv, bs, d // 4)
                        for _ in range(2)) for _ in range(NKV)]
        kc, vc = caches[0]
        qp = feather.pack_fp8_tensor(randn(n_seq * Hq * d).half(), mode="E4M3").view(n_seq, Hq, d // 4)
        bt = torch.randperm(nblk, generator=g, device=dev).to(torch.int32).view(n_seq, cmax // bs)
        for c in (512, 4096):
            cl = torch.full((n_seq,), c, dtype=torch.int32, device=dev)
            us = gpu_time_graph_us(lambda i: paged_attention_fp8_acc_fp32_gpu(qp, caches[i % NKV][0], caches[i % NKV][1], bt, cl,
                                                                              mode="E4M3", max_context_len=c), 16, sync)
            extra[f"paged_attn_e4m3_s32_h32kv4_d64_ctx{c}_us"] = round(us, 2)
            extra[f"paged_attn_e4m3_s32_h32kv4_d64_ctx{c}_GBps"] = round(2 * n_seq * Hkv * d * c / us / 1e3, 1)
            rl[f"paged_attn_e4m3_ctx{c}"] = roofline_record(
                ttab, f"paged_attn_e4m3_ctx{c}", "paged_attn_split_kernel<64, E4M3>" + (" + paged_attn_merge_kernel" if c > 512 else ""),
                2 * n_seq * Hkv * d * c + n_seq * Hq * d * 5, us, launches_per_call=2 if c > 512 else 1, timing="graph",
                note=f"{NKV} K/V cache pairs rotated" + ("" if c > 512 else
                     ": at this context a call reads 8 MB, so the four caches together (34 MB) stay in the 256 MB Infinity Cache"))
        # prefill -> paged cache: 32 sequences x 2048 rows x 4 KV heads of packed K and V (1 B in + 1 B out per code)
        from feather_amd.routines.paged_attention import paged_cache_write
        rows = n_seq * 2048
        ksrc, vsrc = (feather.pack_fp8_tensor(randn(Hkv * rows * d).half(), mode="E4M3").view(Hkv, rows, d // 4)
                      for _ in range(2))
        cu = torch.arange(0, rows + 1, 2048, dtype=torch.int32, device=dev)
        us = gpu_time_graph_us(lambda i: paged_cache_write(ksrc, vsrc, kc, vc, bt, cu, mode="E4M3"), 16, sync)   # device time (graph replay)
        extra["paged_cache_write_e4m3_s32_L2048_kv4_d64_us"] = round(us, 2)
        extra["paged_cache_write_e4m3_s32_L2048_kv4_d64_GBps"] = round(4 * Hkv * rows * d / us / 1e3, 1)
        del kc, vc, caches, qp, ksrc, vsrc
        torch.cuda.empty_cache()
        # decode step of a TinyLlama-1.1B-shaped model (random weights), contexts 512..4095: batch 32 in E4M3
        # (the configuration of the metric), then E5M2 and batch 64 for comparison
        from feather_amd.routines.decode import TINYLLAMA_1_1B as cfg, PackedDecoder, random_weights
        for batch, mode in ((32, "E4M3"), (32, "E5M2"), (64, "E4M3")):
            nb_ = batch * cmax // bs
            wts = random_weights(cfg, seed=5, device=dev)
            dec = PackedDecoder(cfg, wts, n_blocks=nb_, max_blocks=cmax // bs, mode=mode, device=dev)
            del wts
            for lay in dec.layers:
                for name in ("k_cache", "v_cache"):
                    vals = randn(nb_ * cfg.n_kv_heads * bs * cfg.head_dim).half()
                    lay[name].view(-1).copy_(feather.pack_fp8_tensor(vals, mode=mode).view(torch.int32))
            gd = torch.Generator(device=dev).manual_seed(100 + batch)   # the step's own draw: the same contexts in every run
            btd = torch.randperm(nb_, generator=gd, device=dev).to(torch.int32).view(batch, cmax // bs)
            cl = torch.randint(512, cmax, (batch,), generator=gd, device=dev, dtype=torch.int32)
            tok = torch.randint(0, cfg.vocab, (batch,), generator=gd, device=dev, dtype=torch.int32)
            logits = torch.empty((batch, cfg.vocab), dtype=torch.float32, device=dev)
            us = gpu_time_us(lambda i: dec.step(tok, btd, cl, out=logits), 20, 10, sync, warm_ms)
            step_bytes = dec.weight_bytes() + int(cl.sum().item()) * 2 * cfg.n_kv_heads * cfg.head_dim * cfg.n_layers
            key = f"decode_tinyllama_b{batch}_{mode.lower()}"
            extra[key + "_ms_per_step"] = round(us / 1e3, 3)
            extra[key + "_tokens_per_s"] = round(batch / us * 1e6, 0)
            extra[key + "_GBps"] = round(step_bytes / us / 1e3, 1)
            rl[key] = roofline_record(ttab, key, "feather_decode_step (all kernels of one step)", step_bytes, us,
                                      launches_per_call=8 * cfg.n_layers + 3)
            del dec, logits, btd
            torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        from oracle import cpu_baseline
        r = cpu_baseline.gemv_baseline(M, K, "E4M3", sample_rows=M, repeats=5)   # the whole workload, nothing scaled
        cpu = {"value": round(r["total_s"] * 1e6, 1), "unit": "us", "cores": r["cores"], "kind": "port",
               "sample": r["sample"] + "; pack (torch-CPU float8 cast + byte assembly) + decode (LUT gather) + fp32 torch.mv, summed",
               "pack_us": round(r["pack_s"] * 1e6, 1), "decode_us": round(r["decode_s"] * 1e6, 1),
               "compute_us": round(r["compute_s"] * 1e6, 1), "cpu_count": r["cpu_count"]}
        # second half of the metric: pack + decode + fp32 SDPA per head (B4 H16 d=64 L=8192, E5M2), 16 of the 64 heads timed
        def attn_leg(heads, L, d, mode, sample_heads, repeats):
            ra = cpu_baseline.attention_baseline(heads, L, d, mode, sample_heads=sample_heads, repeats=repeats)
            return {"value": round(ra["total_s"] * 1e6, 1), "unit": "us", "cores": ra["cores"], "kind": "port",
                    "sample": ra["sample"] + f"; pack + decode (LUT gather) + fp32 SDPA per head, summed, median of {repeats}",
                    "pack_us": round(ra["pack_s"] * 1e6, 1), "decode_and_sdpa_us": round(ra["compute_s"] * 1e6, 1)}
        cpu["flash_attn_e5m2_b4h16_d64_L8192"] = attn_leg(64, 8192, 64, "E5M2", 16, 3)
        if not args.no_extra:
            # the other configurations, each a bounded sample of the same workload (the scaling is in `sample`)
            r1 = cpu_baseline.gemv_baseline(8192, 8192, "E5M2", sample_rows=8192, repeats=5)
            cpu["gemv_e5m2_8192"] = {"value": round(r1["total_s"] * 1e6, 1), "unit": "us", "cores": r1["cores"], "kind": "port",
                                     "sample": r1["sample"], "pack_us": round(r1["pack_s"] * 1e6, 1),
                                     "decode_us": round(r1["decode_s"] * 1e6, 1), "compute_us": round(r1["compute_s"] * 1e6, 1)}
            rd = cpu_baseline.dot_baseline(1 << 24, "E4M3", repeats=5)
            cpu["dot_e4m3_2p24"] = {"value": round(rd["total_s"] * 1e6, 1), "unit": "us", "cores": rd["cores"], "kind": "port",
                                    "sample": rd["sample"], "pack_us": round(rd["pack_s"] * 1e6, 1),
                                    "decode_us": round(rd["decode_s"] * 1e6, 1), "compute_us": round(rd["compute_s"] * 1e6, 1)}
            cpu["flash_attn_e5m2_b4h16_d64_L4096"] = attn_leg(64, 4096, 64, "E5M2", 16, 3)
            cpu["flash_attn_e4m3_b1h8_d256_L4096"] = attn_leg(8, 4096, 256, "E4M3", 8, 3)
            cpu["flash_attn_e4m3_b1h8_d512_L8192"] = attn_leg(8, 8192, 512, "E4M3", 2, 3)
            from feather_amd.routines.decode import TINYLLAMA_1_1B
            gcpu = torch.Generator().manual_seed(5)
            rs = cpu_baseline.decode_step_baseline(TINYLLAMA_1_1B, 32, torch.randint(512, 4096, (32,), generator=gcpu).tolist(),
                                                   "E4M3", sample_layers=2, repeats=3)
            cpu["decode_tinyllama_b32_e4m3"] = {"value": round(rs["total_s"] * 1e3, 2), "unit": "ms per step", "cores": rs["cores"],
                                                "kind": "port", "sample": rs["sample"],
                                                "tokens_per_s": round(32 / rs["total_s"], 1)}

    line = {
        "metric": "packed-FP8 GEMV us (16384^2, E4M3, FP32 accumulate)",
        "value": round(kern_us, 3), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "E4M3 packed GEMV 16384x16384 + vector 16384 (the configuration the metric is quoted on); N(0,1) fp16 "
                               "sources with 1% of entries x1e-3, packed 4 codes per 32-bit word; 4 distinct "
                               "matrices (1 GiB) rotated",
                   "M": M, "K": K, "mode": "E4M3", "buffers": NBUF, "clock_prewarm_launches": PREWARM, "gate_launches": GATE},
        # the headline kernel's record; the second half of the metric (flash attention d = 64, L = 8192) is the nested
        # matrix-core record, the other attention workloads are in extra.roofline_mfma
        "roofline": dict(headline, avg_launch_us=round(kern_us, 3),
                         **({"flash_attn_e5m2_b4h16_d64_L8192": arl["flash_attn_e5m2_b4h16_d64_L8192"]}
                            if "flash_attn_e5m2_b4h16_d64_L8192" in arl else {})),
        "cpu_baseline": cpu,
        "extra": dict(extra, roofline=rl, roofline_mfma=arl),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
