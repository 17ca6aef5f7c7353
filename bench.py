#!/usr/bin/env python3
"""Benchmark of the hot path: Q4_K dequantize-GEMV 1 x 4096 -> 14336 on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one call of the quantized matmul (m = 1) over one weight matrix.  The weights
rotate over 16 distinct copies (528 MB) so that no cache level can serve them: every step
streams its 33 MB from HBM.  The K timed steps are enqueued from one C call on one stream
and bracketed by events on that stream.  Prints one JSON line.
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

N, K_DIM, M = 14336, 4096, 1
DTYPE = 12  # GGML Q4_K
COPIES = 16
HBM_PEAK_GBS = 8000.0


# HBM bytes per launch of the timed kernel on this workload, from two counter passes
# (FETCH_SIZE 16,249.5 KiB and WRITE_SIZE 56.0 KiB per dispatch) scaled by what the same
# counters read for a plain 32,256 KiB copy kernel (factors 1.9986 and 1.0000).
TRAFFIC_BYTES_PER_LAUNCH = 33_312_900


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def device_weights(torch, n_rows: int, k: int, copies: int):
    """Random Q4_K matrices generated on the device: uniform packed bytes, f16 d/dmin in (0.001, 0.05)."""
    from gllm_amd.ggml import row_bytes
    total = n_rows * row_bytes(DTYPE, k)
    out = []
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    for _ in range(copies):
        w = torch.randint(0, 256, (total,), dtype=torch.uint8, device="cuda", generator=g)
        blocks = w.view(-1, 144)
        d = (torch.rand(blocks.shape[0], 2, device="cuda", generator=g) * 0.049 + 0.001).to(torch.float16)
        blocks[:, 0:4] = d.view(torch.uint8).view(-1, 4)
        out.append(w)
    return out


def cpu_baseline(budget_s: float = 12.0):
    """The oracle's reference-faithful matmul (per-block decode, f32 multiply-add) on the host
    cores, on the same shape with the same generator, repeated for about `budget_s` seconds."""
    from gllm_amd.ggml import row_bytes
    from gllm_amd.synth import random_activations, random_weight
    from oracle import cref
    threads = max(1, min(os.cpu_count() or 1, 16))
    w = random_weight(DTYPE, N, K_DIM, seed=0)
    x = random_activations(M, K_DIM, seed=0)
    cref.quantized_matmul(w, x, DTYPE, M, N, K_DIM, acc=cref.ACC_F32, threads=threads)
    reps, t0 = 0, time.perf_counter()
    while True:
        cref.quantized_matmul(w, x, DTYPE, M, N, K_DIM, acc=cref.ACC_F32, threads=threads)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or reps >= 2000:
            break
    bytes_per_call = N * row_bytes(DTYPE, K_DIM) + M * K_DIM * 4 + M * N * 4
    return {"value": round(bytes_per_call * reps / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "us_per_call": round(dt / reps * 1e6, 1),
            "sample": f"{reps} calls of the same 1x{K_DIM}x{N} Q4_K matmul (C restatement of the reference's "
                      f"scalar decode + f32 FMA, rows split over {threads} threads) in {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-context", action="store_true",
                    help="skip the cache-resident and streaming-read context runs (profiling: only the timed kernel launches)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch plain device-to-device copies of one 33 MB weight buffer (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build measures one GPU; the quantized matmul path has no multi-GPU part "
            "(rows would shard by N with no collective). Run with --gpus 1.")
        sys.exit(2)

    import torch

    from gllm_amd.backend import HipBackend
    from gllm_amd.ggml import row_bytes

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    hip = HipBackend(0)
    ws = device_weights(torch, N, K_DIM, COPIES)
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    x = torch.randn(M, K_DIM, device="cuda", generator=g)
    ys = [torch.empty(M, N, device="cuda") for _ in range(COPIES)]
    nb = ws[0].numel()
    bytes_per_call = N * row_bytes(DTYPE, K_DIM) + M * K_DIM * 4 + M * N * 4  # 33,103,872

    def descs(count, single=False):
        return [(ws[0 if single else i % COPIES], x, ys[0 if single else i % COPIES], DTYPE, M, N, K_DIM)
                for i in range(count)]

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(batch):
        torch.cuda.synchronize()
        start.record()
        hip.quantized_matmul_batch(batch)
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop)  # ms

    if args.copy_probe:
        # A plain copy kernel of known size: 33,030,144 bytes read and as many written per launch.
        dst = torch.empty_like(ws[0])
        for i in range(8):
            dst.copy_(ws[i % COPIES])
        torch.cuda.synchronize()
    hip.quantized_matmul_batch(descs(args.warmup))
    torch.cuda.synchronize()
    ms = timed(descs(args.steps))
    us_per_call = ms * 1e3 / args.steps
    gbs = bytes_per_call / (us_per_call * 1e-6) / 1e9

    # context figures (stderr): cache-resident weights, and the device's streaming-read rate
    context = None
    if not args.no_context:
        ms1 = timed(descs(min(args.steps, 1000), single=True))
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        for i in range(32):
            hip.stream_read(ws[i % COPIES], sink)
        torch.cuda.synchronize()
        start.record()
        for i in range(400):
            hip.stream_read(ws[i % COPIES], sink)
        stop.record()
        torch.cuda.synchronize()
        probe_us = start.elapsed_time(stop) * 1e3 / 400
        context = {"cache_resident_us_per_call": round(ms1 * 1e3 / min(args.steps, 1000), 3),
                   "stream_read_probe_gbs": round(nb / probe_us / 1e3, 1)}
    log(f"Q4_K GEMV 1x{K_DIM}x{N}: {us_per_call:.2f} us/call, {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS * 100:.1f}% of 8 TB/s), "
        f"{2 * N * K_DIM / (us_per_call * 1e-6) / 1e12:.2f} TFLOP/s")
    if context:
        log(f"  same weights every call (cache resident): {context['cache_resident_us_per_call']:.2f} us/call")
        log(f"  streaming-read probe over the same 33 MB buffers: {context['stream_read_probe_gbs']:.0f} GB/s")

    result = {
        "metric": "Q4_K GEMV 1x4096x14336: achieved HBM GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_call / 1e3, 6),
        "us_per_call": round(us_per_call, 3),
        "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 2),
        "tflops": round(2 * N * K_DIM / (us_per_call * 1e-6) / 1e12, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": f"Q4_K dequant-GEMV M=1 K={K_DIM} N={N} (GGUF 144-byte super-blocks), f32 activations "
                               f"~N(0,1) as 23-bit block fixed point, int8 MFMA with i32 accumulation, f32 scales; "
                               f"weights rotate over {COPIES} copies ({COPIES * nb >> 20} MiB) so every call reads HBM",
                   "bytes_per_call": bytes_per_call, "kernel": "gq_mm8_q4k_p1_e1"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH,
                     "note": "achieved = 33,103,872 algorithmic bytes / (event time over the timed region / steps); "
                             "the event time includes the gap between back-to-back launches"},
    }
    if context:
        result["context"] = context
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
        log(f"  CPU baseline: {result['cpu_baseline']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
