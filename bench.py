#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Headline (one JSON line on stdout): fp16 GEMM M = N = K = 4096, A row-major, B column-major,
fp32 accumulate, fp16 output -- TFLOP/s, with the roofline of that kernel and the CPU oracle
timed next to it.  The other kernels of the path (fp32 GEMM 2048^3, Zamba2-shaped causal conv1d +
SiLU, causal softmax 32 x 2048 x 2048, Gemma2 softmax 8 x 8192 x 8192 with softcap and sliding
window, and the callers either side: fused attention, decode attention, gated RMS norm, the Gemma2
output head at 8 rows) are measured in the same run and reported under "kernels", each with its own roofline object and,
for the configurations the metric names, the CPU oracle timed on a bounded sample.

A step is one launch of the kernel over one batch of synthetic input that is already resident
in HBM.  Inputs are drawn on the host by anygpu_amd.synth with the stated seeds (the generator of
the parity tests; the 2.4 GB of output-head weights by torch's generator on the device).  Timing of every kernel:
  * W untimed warm-up steps, then exactly K steps between two device synchronisations (host
    clock -> `value` of the headline) and between two HIP events recorded on the launch stream
    (-> `us_per_launch`, `roofline.achieved`); for the kernels under "kernels", whose K is a
    fraction of --steps, K is never below 100 and W never below 10;
  * then the same number of launches (at least 100, at most 200) with an event pair around every
    single launch -> `median_us`, `min_us` (these leave out the gap between two launches, and
    take in the events' own cost), and 25 groups of 8 back-to-back launches under one event
    pair each -> `median_of_8_us` (the median with an eighth of that cost).
The memory-bound kernels rotate over several buffer sets so that the working set exceeds the
256 MB Infinity Cache.

`--gemm-shapes` (or `--gemm-shapes f32`) prints, instead of the JSON line, a table of the fp16 (fp32) GEMM over the
projection shapes of the models the path serves (8 row counts x 14 weight shapes, weights k-contiguous) next to torch.matmul, i.e. the vendor library,
on the same operands; with `--gemm-rows between` 22 row counts between the tile heights (3 .. 2060) over 8 of the
shapes, with `--gemm-layout kn` the weights stored [K, N].

`--attention-shapes` prints a table of the attention forms away from the benchmark's block (generation steps with 1 - 16
queries per head, chunks of 32 - 1024 queries against a cache of 4096 and 32768 keys, causal prompts of a few thousand
tokens; fp16 and fp32, head dimensions 64 / 128 / 256, grouped heads) next to torch's scaled_dot_product_attention on the
same operands, and of the softmax with a mask tensor next to torch.softmax(x * alpha + mask).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time
from pathlib import Path

REPO = Path(__file__).resolve().parent
if str(REPO) not in sys.path:
    sys.path.insert(0, str(REPO))

PEAK_CLOCK_GHZ = 2.4
FP16_FLOP_PER_CLK_PER_CU = 4096
PEAK_FP16_TFLOPS = 2516.6      # dense fp16 MFMA, 256 CU x 4096 flop/clk/CU x 2.4 GHz
PEAK_FP32_TFLOPS = 157.3       # fp32 matrix path
PEAK_HBM_GBS = 8000.0          # HBM3E
MIN_TIMED_LAUNCHES = 100       # every kernel under "kernels": at least this many back-to-back launches are timed ...
MIN_WARMUP_LAUNCHES = 10       # ... after at least this many untimed ones (beyond the settle period), whatever --steps says

# Bytes per launch moved behind the L2s: NOT measured by this run.  They come from two rocprofv3 --pmc runs of this
# command (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), scaled by what the same counters read for a plain 256 MiB
# device copy (fetch x 2.000, write x 1.000); the summary each figure is copied from is named beside it.
MEASURED_TRAFFIC = {
    "gemm_f16": (235046242, "profiles/gemm_f16_4096_ring_kernel.md"),
    "gemm_f32": (117654803, "profiles/gemm_f32_2048_kernel.md"),
    "conv1d": (277197415, "profiles/causal_conv1d_silu_zamba2_tile_kernel.md"),
    "softmax_causal": (406922965, "profiles/softmax_causal_32x2048x2048_window_kernel.md"),
    "softmax_gemma2": (1483615321, "profiles/softmax_gemma2_8x8192x8192_window_kernel.md"),
    "attention_gemma2": (530927292, "profiles/sdp_attention_fwd_f16_gemma2_kernel.md"),
    "attention_gemma2_f32": (1308870403, "profiles/sdp_attention_fwd_f32_gemma2_kernel.md"),
    "gated_rmsnorm": (805405955, "profiles/gated_rmsnorm_f16_row_kernel.md"),
    "attention_decode": (144037358, "profiles/sdp_attention_decode_f16_partial_and_merge_kernels.md"),
    "lm_head_f32": (2391557676, "profiles/gemma_linear_softcap_head_band_kernels.md"),
    "lm_head_f16": (1203714309, "profiles/gemma_linear_softcap_head_band_kernels.md"),
}


def traffic_fields(key):
    nbytes, source = MEASURED_TRAFFIC[key]
    fields = {"traffic": nbytes, "traffic_source": f"{source} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command; copied, not measured in this run)"}
    # which version of the summary the figure was copied from: the file's SHA-1 (the tree that runs here has no history)
    try:
        import hashlib
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), source), "rb") as f:
            fields["traffic_source_sha1"] = hashlib.sha1(f.read()).hexdigest()[:12]
    except OSError:
        fields["traffic_source_sha1"] = None
    return fields


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="target wall time of the CPU-oracle sample of the headline (0 disables every CPU baseline); "
                         "the other configurations get a quarter of it each")
    ap.add_argument("--only", default="", help="comma list of: gemm,gemm32,conv,softmax,attn,attn32,attnmask,decode,norm,head (default: all)")
    ap.add_argument("--gemm-shapes", nargs="?", const="f16", default=None, choices=("f16", "f32"),
                    help="print the table of GEMM layer shapes (fp16, or fp32 with `--gemm-shapes f32`) against torch.matmul and exit")
    ap.add_argument("--attention-shapes", nargs="?", const="all", default=None, choices=("all", "mask_tensor"),
                    help="print the table of attention shapes (generation steps, chunks of a prompt against a cache, masked "
                         "softmax) against torch and exit; `--attention-shapes mask_tensor`: only the attention with the mask "
                         "as a tensor (fused kernel, three launches, torch)")
    ap.add_argument("--gemm-rows", default="layer", choices=("layer", "between"),
                    help="with --gemm-shapes: the row counts of the layer table (powers of two, default) or 22 row counts between "
                         "the tile heights over 8 of the shapes")
    ap.add_argument("--gemm-layout", default="nk", choices=("nk", "kn"),
                    help="with --gemm-shapes: weights stored [N, K] (default) or [K, N]")
    ap.add_argument("--gemm-operands", default="uniform", choices=("uniform", "low_toggle"),
                    help="operands of the headline GEMM: U(-1, 1) as the metric names them (default), or integers -2 .. 2 "
                         "(few bits toggle: for profiler runs of the power-limit comparison; the line then says so)")
    ap.add_argument("--skip-low-toggle", action="store_true",
                    help="leave out the headline's second leg on low-toggle operands (for profiler runs that must see one operand set only)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain device copy of 256 MiB (read 256 MiB + write 256 MiB) a few times, "
                         "as the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counter readings")
    return ap.parse_args()


SETTLE_SECONDS = 0.3


def timed_region(torch, fn, steps, warmup, floor=MIN_TIMED_LAUNCHES):
    """Timing of `fn`: a dict with the host and event time of `steps` back-to-back calls (after the settle period and
    `warmup` untimed calls) and the median / minimum of per-launch event pairs.

    Before the warm-up the kernel runs untimed for SETTLE_SECONDS: after an idle period the
    power management of the GPU over- and undershoots for some tens of milliseconds (a 4096^3
    GEMM takes 124 us, then up to 160 us, then settles near 95 us after about 150 launches), and
    the number that matters for a long-running job is the settled one."""
    steps = max(int(steps), floor)
    if floor > 1:
        warmup = max(int(warmup), MIN_WARMUP_LAUNCHES)
    t_end = time.perf_counter() + SETTLE_SECONDS
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    singles = min(max(steps, MIN_TIMED_LAUNCHES), 200)
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(singles)]
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    each = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
    # an event pair around ONE launch also times the events themselves and a start without a predecessor to overlap
    # (a few microseconds, which is a tenth of the shortest kernels here); the median over groups of 8 back-to-back
    # launches, each group under one pair, carries an eighth of that
    groups = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(25)]
    for a, b in groups:
        a.record()
        for _ in range(8):
            fn()
        b.record()
    torch.cuda.synchronize()
    grouped = sorted(a.elapsed_time(b) * 1e3 / 8 for a, b in groups)
    return {"steps": steps, "warmup": warmup, "host_s": t1 - t0, "event_s": start.elapsed_time(stop) * 1e-3,
            "us_per_launch": start.elapsed_time(stop) * 1e3 / steps,
            "median_us": statistics.median(each), "min_us": each[0], "single_launches": singles,
            "median_of_8_us": statistics.median(grouped)}


def timing_fields(t):
    return {"us_per_launch": t["us_per_launch"], "median_us": t["median_us"], "min_us": t["min_us"], "median_of_8_us": t["median_of_8_us"],
            "timed_launches": t["steps"], "warmup_launches": t["warmup"], "single_launches": t["single_launches"]}


def sized_sample(run, unit_cost_probe, total_units, target_seconds):
    """Run `run(units)` on as many units as fit `target_seconds`, sized from a short probe; (units, seconds)."""
    probe_units = max(1, unit_cost_probe)
    t0 = time.perf_counter()
    run(probe_units)
    per_unit = (time.perf_counter() - t0) / probe_units
    units = int(max(probe_units, min(total_units, target_seconds / max(per_unit, 1e-9))))
    t0 = time.perf_counter()
    run(units)
    return units, time.perf_counter() - t0


# ---------------------------------------------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------------------------------------------

def gemm_f16_clock_probe(torch, capi, a, bt, c, n):
    """The clock the part sustains under the 256 x 256 tile kernel on these operands and the matrix cores' share of those
    cycles, from the kernel's own counters (anygpu_gemm_f16_f32acc_probe): launched back to back for a settle period,
    the last launch read."""
    lib = capi.load()
    tiles = (n // 256) ** 2
    probe = torch.zeros((tiles, 4), dtype=torch.int64, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    t_end = time.perf_counter() + SETTLE_SECONDS
    while time.perf_counter() < t_end:
        for _ in range(20):
            capi.check("anygpu_gemm_f16_f32acc_probe",
                       lib.anygpu_gemm_f16_f32acc_probe(a.data_ptr(), bt.data_ptr(), c.data_ptr(), n, n, n, n, n, n,
                                                        capi.B_COL_MAJOR, probe.data_ptr(), stream))
        torch.cuda.synchronize()
    p = probe.cpu().double()
    cycles, ns = p[:, 1] - p[:, 0], (p[:, 3] - p[:, 2]) * 10.0
    per_xcd = [float(ns[x::8].mean() / 1e3) for x in range(8)]          # tile b runs on XCD b % 8
    return {"sustained_clock_ghz": float((cycles / ns).mean()), "mfma_busy_in_main_loop": float(((n // 32) * 64 * 16 / cycles).mean()),
            "main_loop_us_mean": float(ns.mean() / 1e3), "main_loop_us_max": float(ns.max() / 1e3),
            "main_loop_us_min": float(ns.min() / 1e3), "main_loop_us_slowest_xcd": max(per_xcd), "main_loop_us_fastest_xcd": min(per_xcd)}


def bench_gemm_f16(torch, ops, capi, synth, steps, warmup, operands="uniform", low_toggle_leg=True):
    n = 4096
    if operands == "low_toggle":
        a = torch.from_numpy(synth.integers(0, (n, n), -2, 2).astype("float16")).cuda()
        bt = torch.from_numpy(synth.integers(1, (n, n), -2, 2).astype("float16")).cuda()
    else:
        a = torch.from_numpy(synth.uniform(0, (n, n)).astype("float16")).cuda()
        bt = torch.from_numpy(synth.uniform(1, (n, n)).astype("float16")).cuda()   # B stored [N, K]
    c = torch.empty((n, n), dtype=torch.float16, device="cuda")
    # (the headline times exactly --steps launches; only the kernels below are floored)
    t = timed_region(torch, lambda: ops.tensor_mm(a, bt, out=c, b_layout=capi.B_COL_MAJOR), steps, warmup, floor=1)
    flops = 2.0 * n ** 3
    # the vendor library on the same operands, timed the same way (torch.matmul = hipBLASLt): for scale, not the target
    t_vendor = timed_region(torch, lambda: torch.matmul(a, bt.t(), out=c), steps, warmup, floor=1)
    clock = gemm_f16_clock_probe(torch, capi, a, bt, c, n)
    clock["source"] = ("s_memtime / s_memrealtime around the main loop of every tile (anygpu_gemm_f16_f32acc_probe), "
                       "last launch of a settle period of back-to-back launches after the timed region")
    # The same launch on operands that toggle few bits (integers -2 .. 2, same shapes, layout, kernel and launch
    # count): the matrix cores do the same number of operations, the data paths switch less, the part draws less
    # power and holds a higher clock.  What this run gains over the U(-1, 1) run is what the power limit takes.
    low_toggle = None
    if low_toggle_leg:
        a_lo = torch.from_numpy(synth.integers(0, (n, n), -2, 2).astype("float16")).cuda()
        bt_lo = torch.from_numpy(synth.integers(1, (n, n), -2, 2).astype("float16")).cuda()
        floor_lo = 1 if steps >= MIN_TIMED_LAUNCHES else MIN_TIMED_LAUNCHES
        t_lo = timed_region(torch, lambda: ops.tensor_mm(a_lo, bt_lo, out=c, b_layout=capi.B_COL_MAJOR), steps, warmup, floor=floor_lo)
        t_vendor_lo = timed_region(torch, lambda: torch.matmul(a_lo, bt_lo.t(), out=c), steps, warmup, floor=floor_lo)
        clock_lo = gemm_f16_clock_probe(torch, capi, a_lo, bt_lo, c, n)
        del a_lo, bt_lo
        low_toggle = {"us": t_lo["us_per_launch"], "median_us": t_lo["median_us"], "vendor_us": t_vendor_lo["us_per_launch"],
                      "timed_launches": t_lo["steps"], "clock": clock_lo}
    return {
        "timing": t, "flops": flops,
        "tflops_host": flops * t["steps"] / t["host_s"] / 1e12,
        "tflops_event": flops * t["steps"] / t["event_s"] / 1e12,
        "operands": (a, bt),
        "vendor": {"what": "torch.matmul (hipBLASLt) on the same operands, timed the same way right after",
                   "us_per_launch": t_vendor["us_per_launch"], "median_us": t_vendor["median_us"], "min_us": t_vendor["min_us"]},
        "clock": clock,
        "low_toggle": low_toggle,
    }


def host_cores(oracle):
    """Threads for the all-cores leg of a CPU baseline: what the oracle's thread pool offers, at most the box's CPU share."""
    return min(oracle.max_threads(), int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16)


def cpu_baseline_gemm(oracle, a32, b_view, target_seconds, what):
    """The oracle's tensor_mm (1 thread, the reference's loop order) on the first R rows of the problem; R is sized from a
    short probe so that the sample takes about `target_seconds`.  Also times rows spread over all host cores."""
    m, k = a32.shape
    n = b_view.shape[1]

    def run(rows, threads=1):
        oracle.tensor_mm(a32[:rows], b_view, threads=threads)

    rows, t1 = sized_sample(run, 2, m, target_seconds)
    flops = 2.0 * rows * n * k
    cores = host_cores(oracle)
    rows_mt = min(m, rows * cores)
    t0 = time.perf_counter()
    run(rows_mt, cores)
    tn = time.perf_counter() - t0
    return {
        "value": flops / t1 / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": f"rows 0..{rows - 1} of C ({rows} x {n} x {k} MACs) of {what}, reference loop order, float32 accumulator, "
                  f"{t1:.1f} s" + ("" if rows == m else "; a row sample, the whole product extrapolates linearly"),
        "all_cores": {"value": 2.0 * rows_mt * n * k / tn / 1e12, "unit": "TFLOP/s", "cores": cores,
                      "sample": f"rows 0..{rows_mt - 1}, outer rows split over {cores} threads, {tn:.1f} s"},
    }


def bench_gemm_f32(torch, ops, synth, steps, warmup, cpu_seconds):
    n = 2048
    a_host, b_host = synth.uniform(0, (n, n)), synth.uniform(1, (n, n))
    a, b = torch.from_numpy(a_host).cuda(), torch.from_numpy(b_host).cuda()
    c = torch.empty((n, n), dtype=torch.float32, device="cuda")
    t = timed_region(torch, lambda: ops.tensor_mm(a, b, out=c), steps, warmup)
    flops = 2.0 * n ** 3
    sec = t["us_per_launch"] * 1e-6
    out = {
        "name": "gemm_f32", "workload": "fp32 GEMM M=N=K=2048, row-major operands, U(-1,1), seeds 0 / 1 (BASELINE.json configs[1], fp32 variant)",
        **timing_fields(t), "value": flops / sec / 1e12, "unit": "TFLOP/s", "dtype": "f32",
        "roofline": {"bound": "mfma", "achieved": flops / sec / 1e12, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / sec / 1e12 / PEAK_FP32_TFLOPS, **traffic_fields("gemm_f32"), "algorithmic_flops": flops},
    }
    if cpu_seconds > 0:
        import oracle
        out["cpu_baseline"] = cpu_baseline_gemm(oracle, a_host, b_host, cpu_seconds, "the same 2048^3 inputs")
    return out


# ---------------------------------------------------------------------------------------------------------------
# conv1d, softmax
# ---------------------------------------------------------------------------------------------------------------

def rotation(torch, first, nbuf):
    """`nbuf` buffer sets for a memory-bound kernel: the seeded tensor and copies of it rolled by whole rows (same
    values at other addresses), so that consecutive launches do not find their input in the Infinity Cache."""
    return [first] + [torch.roll(first, shifts=i, dims=0) for i in range(1, nbuf)]


def quick_us(torch, fn, launches=60, warm=10):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(launches):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e3 / launches


def measure_hbm_ceiling(torch, capi, nbytes=138412032, nbuf=4):
    """What read + write bandwidth this box gives a plain streaming kernel of this library (anygpu_stream_probe:
    dst[i] = src[i], 16-byte accesses), on the working set of the conv1d configuration (138.4 MB read + 138.4 MB written
    per launch, `nbuf` rotating buffer pairs): the best of block sizes {256, 512, 1024} x accesses per lane {1, 2, 4}
    x non-temporal or plain stores, each timed over 60 back-to-back launches after 10 warm-ups; the three best are
    timed again over 200."""
    lib = capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    srcs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_() for _ in range(nbuf)]
    dsts = [torch.empty_like(x) for x in srcs]
    it = [0]

    def runner(block, vpl, nt_store):
        def step():
            i = it[0] % nbuf
            it[0] += 1
            capi.check("anygpu_stream_probe", lib.anygpu_stream_probe(srcs[i].data_ptr(), dsts[i].data_ptr(), nbytes, block, vpl,
                                                                      1, nt_store, 0, stream))
        return step

    sweep = []
    for block in (256, 512, 1024):
        for vpl in (1, 2, 4):
            for nt_store in (1, 0):
                sweep.append((quick_us(torch, runner(block, vpl, nt_store)), block, vpl, nt_store))
    sweep.sort()
    finals = sorted((quick_us(torch, runner(b, v, nt), launches=200, warm=10), b, v, nt) for _, b, v, nt in sweep[:3])
    us, block, vpl, nt_store = finals[0]
    assert torch.equal(srcs[0], dsts[0])
    return {"gbs": 2 * nbytes / us / 1e3, "us_per_launch": us, "frac_of_peak": 2 * nbytes / us / 1e3 / PEAK_HBM_GBS,
            "bytes_read": nbytes, "bytes_written": nbytes, "rotating_buffer_pairs": nbuf,
            "best": {"block": block, "vectors_per_lane": vpl, "nt_stores": bool(nt_store)},
            "worst_gbs": 2 * nbytes / sweep[-1][0] / 1e3,
            "what": "anygpu_stream_probe, dst[i] = src[i] in 16-byte accesses with non-temporal loads: best of block sizes "
                    "{256, 512, 1024} x accesses per lane {1, 2, 4} x non-temporal / plain stores, measured in this run"}


def bench_conv1d(torch, ops, capi, synth, steps, warmup, cpu_seconds):
    import numpy as np
    b, d, s, width = 4, 4224, 4096, 4
    nbuf = 4                                     # 4 x 277 MB of x + y: well past the Infinity Cache
    x_host = synth.normal(0, (b, d, s)).astype(np.float16)
    w_host = synth.normal(1, (d, width), std=0.5).astype(np.float16)
    b_host = synth.normal(2, (d,), std=0.1).astype(np.float16)
    xs = rotation(torch, torch.from_numpy(x_host).cuda(), nbuf)
    ys = [torch.empty_like(x) for x in xs]
    w, bias = torch.from_numpy(w_host).cuda(), torch.from_numpy(b_host).cuda()
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_causal_conv1d(xs[i], w, bias, out=ys[i])

    t = timed_region(torch, step, steps, warmup)
    nbytes = 2 * b * d * s * 2 + d * width * 2 + d * 2
    sec = t["us_per_launch"] * 1e-6
    del xs[1:], ys[1:]
    ceiling = measure_hbm_ceiling(torch, capi, nbytes=b * d * s * 2, nbuf=nbuf)
    out = {
        "name": "causal_conv1d_silu_f16",
        "workload": "Zamba2-1.2B conv1d + SiLU: x fp16 [4, 4224, 4096] N(0,1) seed 0, w [4224, 4] N(0,0.5) seed 1, bias [4224] "
                    "N(0,0.1) seed 2, left pad 3 (BASELINE.json configs[2]); 4 rotating buffer sets",
        **timing_fields(t), "value": nbytes / sec / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / sec / 1e9 / PEAK_HBM_GBS, **traffic_fields("conv1d"), "algorithmic_bytes": nbytes,
                     "frac_on_median": nbytes / (t["median_us"] * 1e-6) / 1e9 / PEAK_HBM_GBS,
                     "frac_on_median_of_8": nbytes / (t["median_of_8_us"] * 1e-6) / 1e9 / PEAK_HBM_GBS,
                     "hbm_ceiling_gbs": ceiling["gbs"], "frac_of_hbm_ceiling": nbytes / sec / 1e9 / ceiling["gbs"]},
        "hbm_ceiling": ceiling,
    }
    if cpu_seconds > 0:
        import oracle
        x32 = oracle.cvt_f16_to_f32(x_host[0])[None]          # batch 0: [1, d, s]
        w32, b32 = oracle.cvt_f16_to_f32(w_host), oracle.cvt_f16_to_f32(b_host)

        def run(chans, threads=1):
            oracle.tensor_causal_conv1d(x32[:, :chans], w32[:chans], b32[:chans], threads=threads)

        chans, sec_cpu = sized_sample(run, 8, d, cpu_seconds)
        sample_bytes = 2 * chans * s * 2 + chans * width * 2 + chans * 2
        cores = host_cores(oracle)
        chans_mt = min(d, chans * cores)
        t0 = time.perf_counter()
        run(chans_mt, cores)
        sec_mt = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": sample_bytes / sec_cpu / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"channels 0..{chans - 1} of batch 0 ({chans} rows of 4096 samples; fp16 inputs up-cast to float32 as the "
                      f"reference's tests do) of the same inputs, {sec_cpu:.1f} s; algorithmic fp16 bytes of those rows over the "
                      f"time, the whole tensor ({b * d} rows) extrapolates linearly",
            "all_cores": {"value": (2 * chans_mt * s * 2 + chans_mt * width * 2 + chans_mt * 2) / sec_mt / 1e9, "unit": "GB/s",
                          "cores": cores, "sample": f"channels 0..{chans_mt - 1} of batch 0, rows split over {cores} threads, {sec_mt:.1f} s"}}
    return out


def bench_softmax(torch, ops, synth, steps, warmup, cpu_seconds, *, name, heads, q, k, std, alpha, cap, window, nbuf, workload, key):
    import numpy as np
    rows = heads * q
    x_host = synth.normal_matrix_f16(0, rows, k, std)
    xs = rotation(torch, torch.from_numpy(x_host).cuda(), nbuf)
    ys = [torch.empty_like(x) for x in xs]
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_softmax(xs[i], out=ys[i], alpha=alpha, softcap=cap, causal=True, window=window, q_len=q)

    t = timed_region(torch, step, steps, warmup)
    dense = 2 * rows * k * 2                        # read every score once, write every probability once
    i = torch.arange(q, dtype=torch.int64)
    visible = torch.minimum(i + 1, torch.tensor(window if window > 0 else q)).sum().item() * heads
    mask_aware = visible * 2 + rows * k * 2         # reads of visible keys only + full write
    sec = t["us_per_launch"] * 1e-6
    out = {
        "name": name, "workload": workload,
        **timing_fields(t), "value": dense / sec / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": dense / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": dense / sec / 1e9 / PEAK_HBM_GBS, **traffic_fields(key),
                     "algorithmic_bytes": dense, "mask_aware_bytes": mask_aware,
                     "mask_aware_gbs": mask_aware / sec / 1e9, "physical_gbs": MEASURED_TRAFFIC[key][0] / sec / 1e9},
    }
    if cpu_seconds > 0:
        import oracle
        # every (rows / n)-th row, so that short and long visible ranges are sampled alike; a row travels alone, with
        # its query index as the diagonal shift
        def run(n):
            idx = np.linspace(0, rows - 1, n).astype(np.int64)
            x32 = oracle.cvt_f16_to_f32(x_host[idx])
            for tt, r in enumerate(idx):
                oracle.attention_softmax(x32[tt:tt + 1], alpha=alpha, softcap=cap, causal=True, window=window, q_len=0, diag=int(r % q))

        n, sec_cpu = sized_sample(run, 16, rows, cpu_seconds)
        # all cores: a run of consecutive rows from the middle of head 0 (the query index travels as the diagonal
        # shift), rows dealt to the threads; the oracle evaluates every column of a row whatever the mask hides
        cores = host_cores(oracle)
        n_mt = int(min(q // 2, max(n * cores, cores)))
        first = q // 2 - n_mt // 2
        x32_mt = oracle.cvt_f16_to_f32(x_host[first:first + n_mt])
        t0 = time.perf_counter()
        oracle.attention_softmax(x32_mt, alpha=alpha, softcap=cap, causal=True, window=window, q_len=0, diag=first, threads=cores)
        sec_mt = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": n * 2 * k * 2 / sec_cpu / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} rows spread evenly over the {rows} of the same inputs (fp16 up-cast to float32; scale, softcap, mask and "
                      f"softmax in the reference's arithmetic: exp in double, sum in float32), {sec_cpu:.1f} s; dense fp16 bytes "
                      f"of those rows over the time, the whole matrix extrapolates linearly",
            "all_cores": {"value": n_mt * 2 * k * 2 / sec_mt / 1e9, "unit": "GB/s", "cores": cores,
                          "sample": f"rows {first}..{first + n_mt - 1} of head 0, rows dealt to {cores} threads, {sec_mt:.1f} s"}}
    return out


# ---------------------------------------------------------------------------------------------------------------
# the callers either side of the path
# ---------------------------------------------------------------------------------------------------------------

def attention_inputs(torch, synth, h, hkv, n, d, dtype):
    q = torch.from_numpy(synth.normal(1, (1, h, n, d)).astype(dtype)).cuda()
    k = torch.from_numpy(synth.normal(2, (1, hkv, n, d)).astype(dtype)).cuda()
    v = torch.from_numpy(synth.normal(3, (1, hkv, n, d)).astype(dtype)).cuda()
    return q, k, v


def bench_attention(torch, ops, synth, steps, warmup, dtype):
    # Gemma2 attention block at the shape of the softmax headline configuration: 8 query heads over 4 key / value
    # heads, 8192 positions, head_dim 256, scale 1 / 16, softcap 50, causal + window 4096, one fused kernel.  fp16, and
    # float32 (the precision the reference runs Gemma2 in: fp32 operands, fp32 MFMA).
    h, hkv, n, d, win = 8, 4, 8192, 256, 4096
    q, k, v = attention_inputs(torch, synth, h, hkv, n, d, "float16" if dtype == "f16" else "float32")
    t = timed_region(torch, lambda: ops.sdp_attention_fwd(q, k, v, 1.0 / 16.0, softcap=50.0, causal=True, window=win), steps, warmup)
    pairs = win * (win + 1) // 2 + (n - win) * win          # visible (query, key) pairs per head
    flops = 4.0 * d * pairs * h                             # q k^T and p v, 2 flop per multiply-add
    sec = t["us_per_launch"] * 1e-6
    peak = PEAK_FP16_TFLOPS if dtype == "f16" else PEAK_FP32_TFLOPS
    return {
        "name": f"sdp_attention_fwd_{dtype}",
        "workload": f"fused attention {'fp16' if dtype == 'f16' else 'fp32'} q [1, 8, 8192, 256], k / v [1, 4, 8192, 256] N(0,1) seeds 1 / 2 / 3, "
                    "x 1/16, softcap 50, causal + window 4096",
        **timing_fields(t), "value": flops / sec / 1e12, "unit": "TFLOP/s", "dtype": dtype,
        "roofline": {"bound": "mfma", "achieved": flops / sec / 1e12, "peak": peak, "unit": "TFLOP/s",
                     "frac": flops / sec / 1e12 / peak,
                     **traffic_fields("attention_gemma2" if dtype == "f16" else "attention_gemma2_f32"),
                     "algorithmic_flops": flops, "visible_pairs_per_head": pairs},
    }


def bench_attention_mask_tensor(torch, ops, synth, steps, warmup, dtype):
    # The reference's own attention interface (sdp_attention_masked_scaled_fwd, srcs/transformers/sdp.hpp:207-274): the
    # mask arrives as a tensor [1, 1, queries, keys], here the causal + sliding-window mask of a Gemma2 local layer
    # (-inf where hidden), shared by 8 heads of 8192 positions, head_dim 256, scale 1 / 16.  One pass over the mask (which
    # key tiles are hidden from which blocks of queries) and one fused kernel that reads the mask as data; timed together.
    h, n, d, win = 8, 8192, 256, 4096
    tdt = torch.float16 if dtype == "f16" else torch.float32
    q, k, v = attention_inputs(torch, synth, h, h, n, d, "float16" if dtype == "f16" else "float32")
    rows = torch.arange(n, device="cuda").reshape(n, 1)
    cols = torch.arange(n, device="cuda").reshape(1, n)
    mask = torch.zeros(n, n, device="cuda", dtype=tdt)
    mask.masked_fill_((cols > rows) | (cols <= rows - win), float("-inf"))
    m4 = mask.reshape(1, 1, n, n)
    t = timed_region(torch, lambda: ops.sdp_attention_masked_scaled_fwd(q, k, v, m4, 1.0 / 16.0), steps, warmup)
    pairs = win * (win + 1) // 2 + (n - win) * win          # visible (query, key) pairs per head
    flops = 4.0 * d * pairs * h
    sec = t["us_per_launch"] * 1e-6
    peak = PEAK_FP16_TFLOPS if dtype == "f16" else PEAK_FP32_TFLOPS
    return {
        "name": f"sdp_attention_mask_tensor_{dtype}",
        "workload": f"attention with the mask as a tensor, {'fp16' if dtype == 'f16' else 'fp32'}: q, k, v [1, 8, 8192, 256] N(0,1) seeds 1 / 2 / 3, x 1/16, "
                    "mask [1, 1, 8192, 8192] causal + window 4096 as 0 / -inf; pass over the mask + fused kernel",
        **timing_fields(t), "value": flops / sec / 1e12, "unit": "TFLOP/s", "dtype": dtype,
        "roofline": {"bound": "mfma", "achieved": flops / sec / 1e12, "peak": peak, "unit": "TFLOP/s",
                     "frac": flops / sec / 1e12 / peak, "traffic": None,
                     "algorithmic_flops": flops, "visible_pairs_per_head": pairs, "mask_bytes": mask.numel() * mask.element_size()},
    }


def bench_attention_decode(torch, capi, synth, steps, warmup):
    # One generation step against a long cache: 64 query heads over 8 key / value heads, 32768 cached positions,
    # head_dim 128, causal.  The split-key decode form through the C ABI with the caller's workspace: two launches
    # (partial results per split, merge), timed together; the bytes are the K and V caches, read once.
    h, hkv, n_k, d = 64, 8, 32768, 128
    lib = capi.load()
    q = torch.from_numpy(synth.normal(1, (1, h, 1, d)).astype("float16")).cuda()
    k = torch.from_numpy(synth.normal(2, (1, hkv, n_k, d)).astype("float16")).cuda()
    v = torch.from_numpy(synth.normal(3, (1, hkv, n_k, d)).astype("float16")).cuda()
    y = torch.empty_like(q)
    need = int(lib.anygpu_sdp_attention_decode_workspace_bytes(h, h // hkv, 1, n_k, d, 1, 0))
    capi.check("anygpu_sdp_attention_decode_workspace_bytes", min(need, 0))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    call = (q.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel(), h, h // hkv, 1, n_k, d,
            1.0 / math.sqrt(d), 0.0, 1, 0, stream)

    def step():
        capi.check("anygpu_sdp_attention_decode_f16", lib.anygpu_sdp_attention_decode_f16(*call))

    t = timed_region(torch, step, steps, warmup)
    nbytes = 2 * hkv * n_k * d * 2 + 2 * h * d * 2
    sec = t["us_per_launch"] * 1e-6
    return {
        "name": "sdp_attention_decode_f16",
        "workload": "decode attention fp16 q [1, 64, 1, 128], k / v [1, 8, 32768, 128], x 1/sqrt(128), causal; partial + merge launches",
        **timing_fields(t), "value": nbytes / sec / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / sec / 1e9 / PEAK_HBM_GBS, **traffic_fields("attention_decode"),
                     "algorithmic_bytes": nbytes, "workspace_bytes": need},
    }


def bench_gated_rmsnorm(torch, ops, synth, steps, warmup):
    # Zamba2-7B Mamba2 mixer: batch 4 x 4096 positions, d_inner 8192
    rows, cols, nbuf = 4 * 4096, 8192, 3                    # 3 x 805 MB of x + z + y: past the Infinity Cache
    xs = rotation(torch, torch.from_numpy(synth.normal(0, (rows, cols)).astype("float16")).cuda(), nbuf)
    zs = rotation(torch, torch.from_numpy(synth.normal(1, (rows, cols)).astype("float16")).cuda(), nbuf)
    w = torch.from_numpy(synth.uniform(2, (cols,), 0.5, 1.5).astype("float16")).cuda()
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_zamba_gated_rmsnorm(xs[i], zs[i], w, cols, 1e-5)

    t = timed_region(torch, step, steps, warmup)
    nbytes = 3 * rows * cols * 2 + cols * 2
    sec = t["us_per_launch"] * 1e-6
    return {
        "name": "gated_rmsnorm_f16", "workload": "gated RMS norm fp16 x, z [16384, 8192] N(0,1) seeds 0 / 1, w [8192] U(0.5,1.5) seed 2, eps 1e-5",
        **timing_fields(t), "value": nbytes / sec / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / sec / 1e9 / PEAK_HBM_GBS, **traffic_fields("gated_rmsnorm"), "algorithmic_bytes": nbytes},
    }


def bench_lm_head(torch, ops, steps, warmup, dtype):
    # The Gemma2 output head: softcap(x W^T, 30) with W [vocab, hidden] = [256000, 2304] as the reference stores it
    # (srcs/models/gemma2/gemma_linsoftcap.cu:11-33), 8 rows of x (a decode step of batch 8, or a prompt's last positions).
    # The weights (2.36 GB in float32, 1.18 GB in half) are streamed once per call: the bound is the memory.
    rows, vocab, hidden = 8, 256000, 2304
    tdt = torch.float32 if dtype == "f32" else torch.float16
    gen = torch.Generator(device="cuda").manual_seed(0)
    w = ((torch.rand((vocab, hidden), device="cuda", generator=gen) * 2 - 1) * 0.05).to(tdt)
    x = (torch.rand((1, rows, hidden), device="cuda", generator=gen) * 2 - 1).to(tdt)

    def step():
        ops.tensor_gemma_linear_softcap(x, w, 30.0)

    t = timed_region(torch, step, steps, warmup)
    esize = 4 if dtype == "f32" else 2
    nbytes = (vocab * hidden + rows * hidden + rows * vocab) * esize
    sec = t["us_per_launch"] * 1e-6
    return {
        "name": f"gemma_linear_softcap_{dtype}",
        "workload": f"Gemma2 output head {dtype}: x [1, 8, 2304] U(-1,1), W [256000, 2304] U(-0.05,0.05) (torch generator on the "
                    "device, seed 0), softcap 30",
        **timing_fields(t), "value": nbytes / sec / 1e9, "unit": "GB/s", "dtype": dtype,
        "roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / sec / 1e9 / PEAK_HBM_GBS, **traffic_fields(f"lm_head_{dtype}"), "algorithmic_bytes": nbytes},
    }


LAYER_WEIGHTS = [(9216, 2304), (18432, 2304), (2304, 9216), (2048, 2304), (1024, 2304), (4096, 2304), (2304, 2048),
                 (2048, 2048), (8192, 2048), (2048, 8192), (4096, 4096), (14336, 4096), (4096, 14336), (6144, 4096)]
LAYER_ROWS = (16, 64, 128, 256, 512, 1024, 2048, 4096)
# row counts between the heights of the tiles and of the few-row kernels' row blocks
BETWEEN_WEIGHTS = [(9216, 2304), (2304, 9216), (4096, 4096), (14336, 4096), (4096, 14336), (8192, 2048), (6144, 4096), (18944, 3584)]
BETWEEN_ROWS = (3, 8, 16, 24, 32, 40, 48, 64, 65, 80, 96, 128, 130, 160, 200, 256, 270, 384, 520, 768, 1100, 2060)


def sweep_gemm_shapes(torch, ops, capi, dtype_name="f16", row_set="layer", layout="nk"):
    """[rows, K] x [N, K]^T for the (N, K) of Gemma2-2B / Zamba2 / Llama-8B-sized projections: microseconds of this
    library and of torch.matmul (hipBLASLt) on the same uniform random operands, each the better of two runs of 40
    back-to-back launches taken alternately.  row_set "between": row counts between the tile heights (3 .. 2060) over 8 of
    the shapes; layout "kn": the weights stored [K, N]."""
    def timed(fn, iters=40, warm=8):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    dtype = torch.half if dtype_name == "f16" else torch.float
    print("| rows | K | N | this library us | torch.matmul us | ratio |")
    print("|---:|---:|---:|---:|---:|---:|")
    ratios = []
    weights, row_counts = (LAYER_WEIGHTS, LAYER_ROWS) if row_set == "layer" else (BETWEEN_WEIGHTS, BETWEEN_ROWS)
    for n, k in weights:
        weight = (torch.rand(n, k, device="cuda") * 2 - 1).to(dtype) if layout == "nk" else (torch.rand(k, n, device="cuda") * 2 - 1).to(dtype)
        for rows in row_counts:
            a = (torch.rand(rows, k, device="cuda") * 2 - 1).to(dtype)
            c = torch.empty(rows, n, device="cuda", dtype=dtype)
            if layout == "nk":
                mine = lambda: ops.tensor_mm(a, weight, out=c, b_layout=capi.B_COL_MAJOR)
                theirs = lambda: torch.matmul(a, weight.t(), out=c)
            else:
                mine = lambda: ops.tensor_mm(a, weight, out=c)
                theirs = lambda: torch.matmul(a, weight, out=c)
            t_mine, t_theirs = timed(mine), timed(theirs)
            t_mine, t_theirs = min(t_mine, timed(mine)), min(t_theirs, timed(theirs))
            ratios.append(t_mine / t_theirs)
            print(f"| {rows} | {k} | {n} | {t_mine:.1f} | {t_theirs:.1f} | {t_mine / t_theirs:.2f} |", flush=True)
    ratios.sort()
    print(f"\n{len(ratios)} shapes: median ratio {statistics.median(ratios):.2f}, worst {ratios[-1]:.2f}, "
          f"{sum(r > 1.10 for r in ratios)} above 1.10, {sum(r > 1.05 for r in ratios)} above 1.05, {sum(r < 0.95 for r in ratios)} below 0.95")


def sweep_attention_shapes(torch, ops):
    """Generation steps, chunks of a prompt against a cache and whole causal prompts through sdp_attention_fwd (which picks
    the decode form, the fused form, and the split of the key range) next to torch's scaled_dot_product_attention with the
    same causal rule as a boolean mask (grouped heads by enable_gqa); then the softmax with a mask tensor shared by the
    heads next to torch.softmax(x * alpha + mask).  Microseconds, the better of two runs of 5 launches each side."""
    import torch.nn.functional as F

    def timed(fn, iters=5, warm=2):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    print("| dtype | batch | heads / kv heads | head dim | queries | keys | this library us | torch SDPA us | ratio |")
    print("|---|---:|---:|---:|---:|---:|---:|---:|---:|")
    ratios = []
    for dtype in (torch.half, torch.float):
        for batch, heads, kv_heads in ((1, 32, 8), (1, 8, 1), (1, 64, 8), (4, 32, 8)):
            for d in (64, 128, 256):
                for n_q in (1, 4, 16, 64, 256, 1024):
                    for n_k in (4096, 32768):
                        q = torch.randn(batch, heads, n_q, d, device="cuda").to(dtype)
                        k = torch.randn(batch, kv_heads, n_k, d, device="cuda").to(dtype)
                        v = torch.randn(batch, kv_heads, n_k, d, device="cuda").to(dtype)
                        alpha = d ** -0.5
                        visible = torch.ones(n_q, n_k, dtype=torch.bool, device="cuda").tril(diagonal=n_k - n_q)
                        mine = lambda: ops.sdp_attention_fwd(q, k, v, alpha, causal=True)
                        theirs = lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=visible, scale=alpha, enable_gqa=True)
                        t_mine, t_theirs = min(timed(mine), timed(mine)), min(timed(theirs), timed(theirs))
                        ratios.append(t_mine / t_theirs)
                        print(f"| {str(dtype)[6:]} | {batch} | {heads} / {kv_heads} | {d} | {n_q} | {n_k} | {t_mine:.1f} | {t_theirs:.1f} | {t_mine / t_theirs:.2f} |", flush=True)
        for heads, n, d in ((32, 1024, 128), (8, 3000, 128), (16, 2048, 64), (8, 5000, 256), (32, 640, 128)):
            q, k, v = (torch.randn(1, heads, n, d, device="cuda").to(dtype) for _ in range(3))
            alpha = d ** -0.5
            mine = lambda: ops.sdp_attention_fwd(q, k, v, alpha, causal=True)
            theirs = lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=alpha)
            t_mine, t_theirs = min(timed(mine), timed(mine)), min(timed(theirs), timed(theirs))
            ratios.append(t_mine / t_theirs)
            print(f"| {str(dtype)[6:]} | 1 | {heads} / {heads} | {d} | {n} | {n} | {t_mine:.1f} | {t_theirs:.1f} | {t_mine / t_theirs:.2f} |", flush=True)
    ratios.sort()
    print(f"\n{len(ratios)} shapes: median ratio {statistics.median(ratios):.2f}, worst {ratios[-1]:.2f}, {sum(r > 1.0 for r in ratios)} above 1.00")
    print("\n| dtype | heads | queries | keys | softmax with mask tensor us | GB/s | without mask us | torch.softmax(x * alpha + mask) us |")
    print("|---|---:|---:|---:|---:|---:|---:|---:|")
    for dtype in (torch.half, torch.float):
        for heads, n_q, n_k in ((32, 1024, 1024), (8, 4096, 4096), (8, 8192, 8192), (16, 2000, 2000), (2, 16384, 16384), (8, 1024, 20000), (4, 64, 100000), (8, 16, 32768)):
            x = torch.randn(heads * n_q, n_k, device="cuda").to(dtype)
            mask = torch.zeros(n_q, n_k, device="cuda").to(dtype)
            mask.masked_fill_(torch.ones(n_q, n_k, device="cuda").triu(n_k - n_q + 1).bool(), float("-inf"))
            masked = lambda: ops.tensor_softmax_masked(x, mask, alpha=0.125, q_len=n_q)
            plain = lambda: ops.tensor_softmax(x, alpha=0.125)
            theirs = lambda: torch.softmax(x.view(heads, n_q, n_k) * 0.125 + mask, dim=-1)
            t_masked, t_plain, t_theirs = min(timed(masked), timed(masked)), min(timed(plain), timed(plain)), min(timed(theirs), timed(theirs))
            gbs = (2 * x.numel() + mask.numel()) * x.element_size() / t_masked / 1e3
            print(f"| {str(dtype)[6:]} | {heads} | {n_q} | {n_k} | {t_masked:.1f} | {gbs:.0f} | {t_plain:.1f} | {t_theirs:.1f} |", flush=True)


def sweep_attention_mask_tensor(torch, ops, capi):
    """sdp_attention_masked_scaled_fwd, the reference's attention interface with the mask as a tensor (a causal -inf mask, or
    a dense bias), through the fused kernel that reads the mask as data, next to the three launches it replaces (batched
    q k^T, softmax with the mask tensor, batched p v), the rule form of the same causal mask and torch's
    scaled_dot_product_attention with the same mask tensor.  Microseconds, the better of two runs of 10 launches."""
    import torch.nn.functional as F

    def timed(fn, iters=10, warm=3):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    print("\n| dtype | heads | queries | keys | head dim | mask | fused with mask tensor us | three launches us | rule form us | torch SDPA with the mask us |")
    print("|---|---:|---:|---:|---:|---|---:|---:|---:|---:|")
    for dtype in (torch.half, torch.float):
        for heads, n_q, n_k, d, kind in ((8, 8192, 8192, 256, "causal"), (32, 1024, 1024, 128, "causal"), (32, 2048, 2048, 64, "causal"),
                                         (8, 16, 8192, 256, "causal"), (16, 512, 8192, 128, "causal"), (8, 4096, 4096, 128, "dense bias"),
                                         (8, 256, 32768, 128, "window 4096"), (8, 1024, 32768, 256, "window 4096")):
            q = torch.randn(1, heads, n_q, d, device="cuda").to(dtype)
            k, v = (torch.randn(1, heads, n_k, d, device="cuda").to(dtype) for _ in range(2))
            window = 4096 if kind.startswith("window") else 0
            if kind == "dense bias":
                mask = torch.randn(n_q, n_k, device="cuda").to(dtype)
            else:
                hidden = torch.ones(n_q, n_k, device="cuda").triu(n_k - n_q + 1).bool()
                if window:
                    hidden |= torch.ones(n_q, n_k, device="cuda").tril(n_k - n_q - window).bool()
                mask = torch.zeros(n_q, n_k, device="cuda").to(dtype)
                mask.masked_fill_(hidden, float("-inf"))
            m4 = mask.reshape(1, 1, n_q, n_k)
            alpha = d ** -0.5

            def three():
                scores = ops.tensor_mm_batched(q[0], k[0], b_layout=capi.B_COL_MAJOR)
                probs = ops.tensor_softmax_masked(scores.reshape(-1, n_k), mask, alpha=alpha, q_len=n_q)
                return ops.tensor_mm_batched(probs.reshape(heads, n_q, n_k), v[0])

            fused = lambda: ops.sdp_attention_masked_scaled_fwd(q, k, v, m4, alpha)
            theirs = lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=m4, scale=alpha)
            t_fused, t_three, t_theirs = min(timed(fused), timed(fused)), min(timed(three), timed(three)), min(timed(theirs), timed(theirs))
            rule = "-"
            if kind != "dense bias":
                by_rule = lambda: ops.sdp_attention_fwd(q, k, v, alpha, causal=True, window=window, decode=False)
                rule = f"{min(timed(by_rule), timed(by_rule)):.1f}"
            print(f"| {str(dtype)[6:]} | {heads} | {n_q} | {n_k} | {d} | {kind} | {t_fused:.1f} | {t_three:.1f} | {rule} | {t_theirs:.1f} |", flush=True)


def sample_gemm_shapes(torch, ops, capi):
    """A few products that do not fill the chip with 256 x 256 tiles, ragged ones, ones the chunk loads cannot fetch and two
    output heads with [K, N] weights and few rows, next to torch.matmul on the same operands: microseconds, the better of two runs of 40 launches each side."""
    def timed(fn, iters=40, warm=10):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    out = []
    for m, n, k, layout in [(2048, 2048, 2048, "col"), (512, 6144, 4096, "col"), (1024, 4096, 4096, "col"), (2048, 4096, 4096, "col"),
                            (4096, 4096, 4096, "row"), (4000, 4000, 4096, "col"), (4096, 4100, 4096, "row"),
                            (16, 256000, 2304, "row"), (64, 128256, 4096, "row")]:
        a = (torch.rand(m, k, device="cuda") * 2 - 1).half()
        b = (torch.rand(n, k, device="cuda") * 2 - 1).half() if layout == "col" else (torch.rand(k, n, device="cuda") * 2 - 1).half()
        c = torch.empty(m, n, device="cuda", dtype=torch.half)
        flag = capi.B_COL_MAJOR if layout == "col" else capi.B_ROW_MAJOR
        mine = lambda: ops.tensor_mm(a, b, out=c, b_layout=flag)
        theirs = lambda: torch.matmul(a, b.t() if layout == "col" else b, out=c)
        t_mine, t_theirs = timed(mine), timed(theirs)
        t_mine, t_theirs = min(t_mine, timed(mine)), min(t_theirs, timed(theirs))
        out.append({"m": m, "n": n, "k": k, "b_stored": "[N, K]" if layout == "col" else "[K, N]",
                    "us": round(t_mine, 1), "torch_matmul_us": round(t_theirs, 1)})
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this path has no multi-GPU component); got --gpus {args.gpus}",
              file=sys.stderr)
        return 2

    import torch
    from anygpu_amd import capi, ops, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the product path)", file=sys.stderr)
        return 1
    capi.load()
    torch.cuda.set_device(0)
    if args.gemm_shapes:
        sweep_gemm_shapes(torch, ops, capi, args.gemm_shapes, args.gemm_rows, args.gemm_layout)
        return 0
    if args.attention_shapes:
        if args.attention_shapes == "all":
            sweep_attention_shapes(torch, ops)
        sweep_attention_mask_tensor(torch, ops, capi)
        return 0
    only = set(filter(None, args.only.split(",")))
    want = lambda name: not only or name in only
    props = torch.cuda.get_device_properties(0)
    cpu_side = args.cpu_seconds / 4.0

    kernels = []
    gemm = None
    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if want("gemm"):
        gemm = bench_gemm_f16(torch, ops, capi, synth, args.steps, args.warmup, args.gemm_operands, not args.skip_low_toggle)
    if want("gemm32"):
        kernels.append(bench_gemm_f32(torch, ops, synth, args.steps // 2, args.warmup, cpu_side))
    if want("conv"):
        kernels.append(bench_conv1d(torch, ops, capi, synth, args.steps, args.warmup, cpu_side))
    if want("softmax"):
        kernels.append(bench_softmax(
            torch, ops, synth, args.steps, args.warmup, cpu_side, name="softmax_causal_f16", key="softmax_causal",
            heads=32, q=2048, k=2048, std=4.0, alpha=1.0 / 8.0, cap=0.0, window=0, nbuf=3,
            workload="causal softmax fp16 [1, 32, 2048, 2048], scores N(0,4) seed 0, scaled by 1/8 in-kernel "
                     "(BASELINE.json configs[3]); 3 rotating buffer sets"))
        kernels.append(bench_softmax(
            torch, ops, synth, args.steps // 4, max(args.warmup // 4, 1), cpu_side, name="softmax_gemma2_f16",
            key="softmax_gemma2", heads=8, q=8192, k=8192, std=16.0, alpha=1.0 / 16.0, cap=50.0, window=4096, nbuf=2,
            workload="Gemma2 softmax fp16 [1, 8, 8192, 8192], N(0,16) seed 0, x 1/16, softcap 50, causal + window 4096 "
                     "(BASELINE.json configs[4]); 2 rotating buffer sets"))
    if want("attn"):
        kernels.append(bench_attention(torch, ops, synth, args.steps // 8, max(args.warmup // 4, 1), "f16"))
    if want("attn32"):
        kernels.append(bench_attention(torch, ops, synth, args.steps // 16, max(args.warmup // 8, 1), "f32"))
    if want("attnmask"):
        kernels.append(bench_attention_mask_tensor(torch, ops, synth, args.steps // 8, max(args.warmup // 4, 1), "f16"))
        kernels.append(bench_attention_mask_tensor(torch, ops, synth, args.steps // 16, max(args.warmup // 8, 1), "f32"))
    if want("decode"):
        kernels.append(bench_attention_decode(torch, capi, synth, args.steps, args.warmup))
    if want("norm"):
        kernels.append(bench_gated_rmsnorm(torch, ops, synth, args.steps // 4, max(args.warmup // 4, 1)))
    if want("head"):
        kernels.append(bench_lm_head(torch, ops, args.steps // 4, max(args.warmup // 4, 1), "f32"))
        kernels.append(bench_lm_head(torch, ops, args.steps // 4, max(args.warmup // 4, 1), "f16"))

    line = {
        "metric": "fp16 GEMM TFLOP/s; conv1d & softmax HBM GB/s (% roofline) on 1 MI355X",
        "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "settle_s": SETTLE_SECONDS,
        "config": {"workload": "fp16 GEMM M=N=K=4096, A row-major, B column-major ([N,K] storage), U(-1,1) inputs (seeds 0 / 1), "
                               "fp32 accumulate on MFMA, fp16 output (BASELINE.json configs[1])"},
        "device": {"name": props.name, "compute_units": props.multi_processor_count, "peak_clock_ghz": PEAK_CLOCK_GHZ},
    }
    if args.gemm_operands != "uniform":
        line["config"]["workload"] = ("NOT the metric's operands: fp16 GEMM M=N=K=4096 on integers -2 .. 2 (--gemm-operands low_toggle), "
                                      "same shapes, layout and kernel; for the power-limit comparison only")
    if gemm is not None:
        t = gemm["timing"]
        line["value"] = gemm["tflops_host"]
        line["ms_per_step"] = t["host_s"] / t["steps"] * 1e3
        clock = gemm["clock"]
        peak_at_clock = props.multi_processor_count * FP16_FLOP_PER_CLK_PER_CU * clock["sustained_clock_ghz"] * 1e9 / 1e12
        line["roofline"] = {"bound": "mfma", "achieved": gemm["tflops_event"], "peak": PEAK_FP16_TFLOPS,
                            "unit": "TFLOP/s", "frac": gemm["tflops_event"] / PEAK_FP16_TFLOPS,
                            **traffic_fields("gemm_f16"), **timing_fields(t),
                            "algorithmic_flops": gemm["flops"], "min_bytes": 3 * 4096 * 4096 * 2,
                            **clock, "peak_at_sustained_clock": peak_at_clock,
                            "frac_at_sustained_clock": gemm["tflops_event"] / peak_at_clock,
                            # scalars: the vendor library (torch.matmul = hipBLASLt) on the same operands in the same run
                            "vendor_us": gemm["vendor"]["us_per_launch"],
                            "vendor_frac": gemm["flops"] / (gemm["vendor"]["us_per_launch"] * 1e-6) / 1e12 / PEAK_FP16_TFLOPS,
                            "vendor_library": gemm["vendor"]}
        lo = gemm["low_toggle"]
        if lo is not None:
            # the same launch of this library and of the vendor's on integers -2 .. 2 (same shapes, layout and kernel)
            lo_tflops = gemm["flops"] / (lo["us"] * 1e-6) / 1e12
            line["roofline"].update({
                "low_toggle_us": lo["us"], "low_toggle_median_us": lo["median_us"],
                "low_toggle_frac": lo_tflops / PEAK_FP16_TFLOPS,
                "low_toggle_clock_ghz": lo["clock"]["sustained_clock_ghz"],
                "low_toggle_mfma_busy_in_main_loop": lo["clock"]["mfma_busy_in_main_loop"],
                "vendor_low_toggle_us": lo["vendor_us"],
                "low_toggle_operands": "integers -2 .. 2 (seeds 0 / 1) in place of U(-1, 1); same kernel, shapes, layout; "
                                       f"{lo['timed_launches']} launches after the settle period and warm-up"})
        line["gemm_f16_other_shapes"] = sample_gemm_shapes(torch, ops, capi)
        if args.cpu_seconds > 0:
            import oracle
            a_dev, bt_dev = gemm["operands"]
            a32 = oracle.cvt_f16_to_f32(a_dev.cpu().numpy())
            bt32 = oracle.cvt_f16_to_f32(bt_dev.cpu().numpy())
            line["cpu_baseline"] = cpu_baseline_gemm(oracle, a32, bt32.T, args.cpu_seconds, "the same 4096^3 inputs")
    line["kernels"] = kernels
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
