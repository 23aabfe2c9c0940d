#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Headline (one JSON line on stdout): fp16 GEMM M = N = K = 4096, A row-major, B column-major,
fp32 accumulate, fp16 output -- TFLOP/s, with the roofline of that kernel and the CPU oracle
timed next to it.  The memory-bound kernels of the same path (Zamba2-shaped causal conv1d +
SiLU, causal softmax 32 x 2048 x 2048, Gemma2 softmax 8 x 8192 x 8192 with softcap and sliding
window) are measured in the same run and reported under "kernels", each with its own roofline
object (dense algorithmic bytes / average launch time against 8 TB/s).

A step is one launch of the kernel over one batch of synthetic input that is already resident
in HBM.  Timing: W untimed warm-up steps, then exactly K steps between two device
synchronisations (host clock -> `value`) and between two HIP events recorded on the launch
stream (-> `roofline.achieved`).  The memory-bound kernels rotate over several buffer sets so
that the working set exceeds the 256 MB Infinity Cache.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time
from pathlib import Path

REPO = Path(__file__).resolve().parent
if str(REPO) not in sys.path:
    sys.path.insert(0, str(REPO))

PEAK_FP16_TFLOPS = 2516.6      # dense fp16 MFMA, 256 CU x 4096 flop/clk/CU x 2.4 GHz
PEAK_FP32_TFLOPS = 157.3       # fp32 matrix path
PEAK_HBM_GBS = 8000.0          # HBM3E

# Bytes per launch moved behind the L2s, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (KiB per
# dispatch), scaled by what the same counters read for a plain 256 MiB device copy (fetch x 2.000,
# write x 1.000); the summaries are under profiles/.
MEASURED_TRAFFIC_BYTES = {"gemm_f16": 234962687, "gemm_f32": 167994164, "conv1d": 277226336,
                          "softmax_causal": 410887952, "softmax_gemma2": 1514268488,
                          "attention_gemma2": 188478908, "attention_gemma2_f32": 887738788, "gated_rmsnorm": 805513216,
                          "attention_decode": 144061440}


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="target wall time of the CPU-oracle sample (0 disables the CPU baseline)")
    ap.add_argument("--only", default="", help="comma list of: gemm,gemm32,conv,softmax,attn,attn32,decode,norm (default: all)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain device copy of 256 MiB (read 256 MiB + write 256 MiB) a few times, "
                         "as the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counter readings")
    return ap.parse_args()


SETTLE_SECONDS = 0.3


def timed_region(torch, fn, steps, warmup):
    """(host seconds, event seconds) for `steps` calls of fn after `warmup` untimed calls.

    Before the warm-up the kernel runs untimed for SETTLE_SECONDS: after an idle period the
    power management of the GPU over- and undershoots for some tens of milliseconds (a 4096^3
    GEMM takes 124 us, then up to 160 us, then settles near 100 us after about 150 launches), and
    the number that matters for a long-running job is the settled one."""
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
    return t1 - t0, start.elapsed_time(stop) * 1e-3


def bench_gemm_f16(torch, ops, capi, synth, steps, warmup):
    n = 4096
    a = torch.from_numpy(synth.uniform(0, (n, n)).astype("float16")).cuda()
    bt = torch.from_numpy(synth.uniform(1, (n, n)).astype("float16")).cuda()   # B stored [N, K]
    c = torch.empty((n, n), dtype=torch.float16, device="cuda")
    host_s, ev_s = timed_region(torch, lambda: ops.tensor_mm(a, bt, out=c, b_layout=capi.B_COL_MAJOR), steps, warmup)
    flops = 2.0 * n ** 3
    return {
        "host_s": host_s, "event_s": ev_s, "flops": flops,
        "tflops_host": flops * steps / host_s / 1e12,
        "tflops_event": flops * steps / ev_s / 1e12,
        "operands": (a, bt),
    }


def bench_gemm_f32(torch, ops, synth, steps, warmup):
    n = 2048
    a = torch.from_numpy(synth.uniform(0, (n, n))).cuda()
    b = torch.from_numpy(synth.uniform(1, (n, n))).cuda()
    c = torch.empty((n, n), dtype=torch.float32, device="cuda")
    host_s, ev_s = timed_region(torch, lambda: ops.tensor_mm(a, b, out=c), steps, warmup)
    flops = 2.0 * n ** 3
    t = ev_s / steps
    return {
        "name": "gemm_f32", "workload": "fp32 GEMM M=N=K=2048, row-major operands, U(-1,1)",
        "us_per_launch": t * 1e6, "value": flops / t / 1e12, "unit": "TFLOP/s", "dtype": "f32",
        "roofline": {"bound": "mfma", "achieved": flops / t / 1e12, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / t / 1e12 / PEAK_FP32_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES["gemm_f32"]},
    }


def bench_conv1d(torch, ops, steps, warmup):
    b, d, s, width = 4, 4224, 4096, 4
    nbuf = 4                                     # 4 x 277 MB of x + y: well past the Infinity Cache
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    xs = [torch.randn((b, d, s), device="cuda", generator=g).half() for _ in range(nbuf)]
    ys = [torch.empty_like(x) for x in xs]
    w = (torch.randn((d, width), device="cuda", generator=g) * 0.5).half()
    bias = (torch.randn((d,), device="cuda", generator=g) * 0.1).half()
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_causal_conv1d(xs[i], w, bias, out=ys[i])

    host_s, ev_s = timed_region(torch, step, steps, warmup)
    nbytes = 2 * b * d * s * 2 + d * width * 2 + d * 2
    t = ev_s / steps
    return {
        "name": "causal_conv1d_silu_f16",
        "workload": "Zamba2-1.2B conv1d + SiLU: x fp16 [4, 4224, 4096], w [4224, 4], bias [4224], left pad 3",
        "us_per_launch": t * 1e6, "value": nbytes / t / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / t / 1e9 / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES["conv1d"],
                     "algorithmic_bytes": nbytes},
    }


def bench_softmax(torch, ops, steps, warmup, *, name, heads, q, k, std, alpha, cap, window, nbuf, workload, key):
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    rows = heads * q
    xs = [(torch.randn((rows, k), device="cuda", generator=g) * std).half() for _ in range(nbuf)]
    ys = [torch.empty_like(x) for x in xs]
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_softmax(xs[i], out=ys[i], alpha=alpha, softcap=cap, causal=True, window=window, q_len=q)

    host_s, ev_s = timed_region(torch, step, steps, warmup)
    dense = 2 * rows * k * 2                        # read every score once, write every probability once
    i = torch.arange(q, dtype=torch.int64)
    visible = torch.minimum(i + 1, torch.tensor(window if window > 0 else q)).sum().item() * heads
    mask_aware = visible * 2 + rows * k * 2         # reads of visible keys only + full write
    t = ev_s / steps
    return {
        "name": name, "workload": workload,
        "us_per_launch": t * 1e6, "value": dense / t / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": dense / t / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": dense / t / 1e9 / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES[key],
                     "algorithmic_bytes": dense, "mask_aware_bytes": mask_aware,
                     "mask_aware_gbs": mask_aware / t / 1e9},
    }


def bench_attention(torch, ops, steps, warmup):
    # Gemma2 attention block at the shape of the softmax headline configuration: 8 query heads over 4 key / value
    # heads, 8192 positions, head_dim 256, scale 1 / 16, softcap 50, causal + window 4096, one fused kernel
    h, hkv, n, d, win = 8, 4, 8192, 256, 4096
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    q = torch.randn((1, h, n, d), device="cuda", generator=g).half()
    k = torch.randn((1, hkv, n, d), device="cuda", generator=g).half()
    v = torch.randn((1, hkv, n, d), device="cuda", generator=g).half()
    host_s, ev_s = timed_region(torch, lambda: ops.sdp_attention_fwd(q, k, v, 1.0 / 16.0, softcap=50.0, causal=True, window=win),
                                steps, warmup)
    pairs = win * (win + 1) // 2 + (n - win) * win          # visible (query, key) pairs per head
    flops = 4.0 * d * pairs * h                             # q k^T and p v, 2 flop per multiply-add
    t = ev_s / steps
    return {
        "name": "sdp_attention_fwd_f16",
        "workload": "fused attention fp16 q [1, 8, 8192, 256], k / v [1, 4, 8192, 256], x 1/16, softcap 50, causal + window 4096",
        "us_per_launch": t * 1e6, "value": flops / t / 1e12, "unit": "TFLOP/s", "dtype": "f16",
        "roofline": {"bound": "mfma", "achieved": flops / t / 1e12, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / t / 1e12 / PEAK_FP16_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES["attention_gemma2"],
                     "algorithmic_flops": flops, "visible_pairs_per_head": pairs},
    }


def bench_attention_f32(torch, ops, steps, warmup):
    # the same block in float32 (the precision the reference runs Gemma2 in): fp32 operands, fp32 MFMA
    h, hkv, n, d, win = 8, 4, 8192, 256, 4096
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    q = torch.randn((1, h, n, d), device="cuda", generator=g)
    k = torch.randn((1, hkv, n, d), device="cuda", generator=g)
    v = torch.randn((1, hkv, n, d), device="cuda", generator=g)
    host_s, ev_s = timed_region(torch, lambda: ops.sdp_attention_fwd(q, k, v, 1.0 / 16.0, softcap=50.0, causal=True, window=win),
                                steps, warmup)
    pairs = win * (win + 1) // 2 + (n - win) * win
    flops = 4.0 * d * pairs * h
    t = ev_s / steps
    return {
        "name": "sdp_attention_fwd_f32",
        "workload": "fused attention fp32 q [1, 8, 8192, 256], k / v [1, 4, 8192, 256], x 1/16, softcap 50, causal + window 4096",
        "us_per_launch": t * 1e6, "value": flops / t / 1e12, "unit": "TFLOP/s", "dtype": "f32",
        "roofline": {"bound": "mfma", "achieved": flops / t / 1e12, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / t / 1e12 / PEAK_FP32_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES["attention_gemma2_f32"],
                     "algorithmic_flops": flops, "visible_pairs_per_head": pairs},
    }


def bench_attention_decode(torch, capi, steps, warmup):
    # One generation step against a long cache: 64 query heads over 8 key / value heads, 32768 cached positions,
    # head_dim 128, causal.  The split-key decode form through the C ABI with the caller's workspace: two launches
    # (partial results per split, merge), timed together; the bytes are the K and V caches, read once.
    h, hkv, n_k, d = 64, 8, 32768, 128
    lib = capi.load()
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    q = torch.randn((1, h, 1, d), device="cuda", generator=g).half()
    k = torch.randn((1, hkv, n_k, d), device="cuda", generator=g).half()
    v = torch.randn((1, hkv, n_k, d), device="cuda", generator=g).half()
    y = torch.empty_like(q)
    need = int(lib.anygpu_sdp_attention_decode_workspace_bytes(h, h // hkv, 1, n_k, d, 1, 0))
    capi.check("anygpu_sdp_attention_decode_workspace_bytes", min(need, 0))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    call = (q.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel(), h, h // hkv, 1, n_k, d,
            1.0 / math.sqrt(d), 0.0, 1, 0, stream)

    def step():
        capi.check("anygpu_sdp_attention_decode_f16", lib.anygpu_sdp_attention_decode_f16(*call))

    host_s, ev_s = timed_region(torch, step, steps, warmup)
    nbytes = 2 * hkv * n_k * d * 2 + 2 * h * d * 2
    t = ev_s / steps
    return {
        "name": "sdp_attention_decode_f16",
        "workload": "decode attention fp16 q [1, 64, 1, 128], k / v [1, 8, 32768, 128], x 1/sqrt(128), causal; partial + merge launches",
        "us_per_launch": t * 1e6, "value": nbytes / t / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / t / 1e9 / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get("attention_decode"),
                     "algorithmic_bytes": nbytes, "workspace_bytes": need},
    }


def bench_gated_rmsnorm(torch, ops, steps, warmup):
    # Zamba2-7B Mamba2 mixer: batch 4 x 4096 positions, d_inner 8192
    rows, cols, nbuf = 4 * 4096, 8192, 3                    # 3 x 805 MB of x + z + y: past the Infinity Cache
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    xs = [torch.randn((rows, cols), device="cuda", generator=g).half() for _ in range(nbuf)]
    zs = [torch.randn((rows, cols), device="cuda", generator=g).half() for _ in range(nbuf)]
    w = (torch.rand((cols,), device="cuda", generator=g) + 0.5).half()
    it = [0]

    def step():
        i = it[0] % nbuf
        it[0] += 1
        ops.tensor_zamba_gated_rmsnorm(xs[i], zs[i], w, cols, 1e-5)

    host_s, ev_s = timed_region(torch, step, steps, warmup)
    nbytes = 3 * rows * cols * 2 + cols * 2
    t = ev_s / steps
    return {
        "name": "gated_rmsnorm_f16", "workload": "gated RMS norm fp16 x, z [16384, 8192], w [8192], eps 1e-5",
        "us_per_launch": t * 1e6, "value": nbytes / t / 1e9, "unit": "GB/s", "dtype": "f16",
        "roofline": {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": nbytes / t / 1e9 / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES["gated_rmsnorm"],
                     "algorithmic_bytes": nbytes},
    }


def cpu_baseline_gemm(a_dev, bt_dev, target_seconds):
    """The oracle's tensor_mm (1 thread, the reference's loop order) on the first R rows of the
    same 4096^3 problem; R is sized from a short probe so that the sample takes about
    `target_seconds`.  Also times the same rows spread over all host cores."""
    import numpy as np
    import oracle

    a = oracle.cvt_f16_to_f32(a_dev.cpu().numpy())
    bt = oracle.cvt_f16_to_f32(bt_dev.cpu().numpy())
    n = a.shape[0]
    b_view = bt.T                                    # column-major B as a strided view

    def run(rows, threads):
        t0 = time.perf_counter()
        oracle.tensor_mm(a[:rows], b_view, threads=threads)
        return time.perf_counter() - t0

    probe_rows = 2
    probe_s = run(probe_rows, 1)
    per_row = probe_s / probe_rows
    rows = int(max(probe_rows, min(n, target_seconds / max(per_row, 1e-9))))
    t1 = run(rows, 1)
    flops = 2.0 * rows * n * n
    cores = min(oracle.max_threads(), int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16)
    rows_mt = min(n, rows * cores)
    tn = run(rows_mt, cores)
    return {
        "value": flops / t1 / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": f"rows 0..{rows - 1} of C ({rows} x {n} x {n} MACs) of the same 4096^3 inputs, "
                  f"reference loop order, float32 accumulator, {t1:.1f} s",
        "all_cores": {"value": 2.0 * rows_mt * n * n / tn / 1e12, "unit": "TFLOP/s", "cores": cores,
                      "sample": f"rows 0..{rows_mt - 1}, outer rows split over {cores} threads, {tn:.1f} s"},
    }


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
    only = set(filter(None, args.only.split(",")))
    want = lambda name: not only or name in only
    props = torch.cuda.get_device_properties(0)

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
        gemm = bench_gemm_f16(torch, ops, capi, synth, args.steps, args.warmup)
    if want("gemm32"):
        kernels.append(bench_gemm_f32(torch, ops, synth, max(args.steps // 2, 1), args.warmup))
    if want("conv"):
        kernels.append(bench_conv1d(torch, ops, args.steps, args.warmup))
    if want("softmax"):
        kernels.append(bench_softmax(
            torch, ops, args.steps, args.warmup, name="softmax_causal_f16", key="softmax_causal",
            heads=32, q=2048, k=2048, std=4.0, alpha=1.0 / 8.0, cap=0.0, window=0, nbuf=3,
            workload="causal softmax fp16 [1, 32, 2048, 2048], scores N(0,4) scaled by 1/8 in-kernel"))
        kernels.append(bench_softmax(
            torch, ops, max(args.steps // 4, 1), max(args.warmup // 4, 1), name="softmax_gemma2_f16",
            key="softmax_gemma2", heads=8, q=8192, k=8192, std=16.0, alpha=1.0 / 16.0, cap=50.0, window=4096, nbuf=2,
            workload="Gemma2 softmax fp16 [1, 8, 8192, 8192], N(0,16) x 1/16, softcap 50, causal + window 4096"))

    if want("attn"):
        kernels.append(bench_attention(torch, ops, max(args.steps // 8, 1), max(args.warmup // 4, 1)))
    if want("attn32"):
        kernels.append(bench_attention_f32(torch, ops, max(args.steps // 16, 1), max(args.warmup // 8, 1)))
    if want("decode"):
        kernels.append(bench_attention_decode(torch, capi, args.steps, args.warmup))
    if want("norm"):
        kernels.append(bench_gated_rmsnorm(torch, ops, max(args.steps // 4, 1), max(args.warmup // 4, 1)))

    line = {
        "metric": "fp16 GEMM TFLOP/s; conv1d & softmax HBM GB/s (% roofline) on 1 MI355X",
        "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "settle_s": SETTLE_SECONDS,
        "config": {"workload": "fp16 GEMM M=N=K=4096, A row-major, B column-major ([N,K] storage), U(-1,1) inputs, "
                               "fp32 accumulate on MFMA, fp16 output (BASELINE.json configs[1])"},
        "device": {"name": props.name, "compute_units": props.multi_processor_count,
                   "clock_mhz": getattr(props, "clock_rate", 0) / 1e3 if hasattr(props, "clock_rate") else None},
    }
    if gemm is not None:
        t_ev = gemm["event_s"] / args.steps
        line["value"] = gemm["tflops_host"]
        line["ms_per_step"] = gemm["host_s"] / args.steps * 1e3
        line["roofline"] = {"bound": "mfma", "achieved": gemm["tflops_event"], "peak": PEAK_FP16_TFLOPS,
                            "unit": "TFLOP/s", "frac": gemm["tflops_event"] / PEAK_FP16_TFLOPS,
                            "traffic": MEASURED_TRAFFIC_BYTES["gemm_f16"], "us_per_launch": t_ev * 1e6,
                            "algorithmic_flops": gemm["flops"], "min_bytes": 3 * 4096 * 4096 * 2}
        if args.cpu_seconds > 0:
            line["cpu_baseline"] = cpu_baseline_gemm(*gemm["operands"], args.cpu_seconds)
    line["kernels"] = kernels
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
