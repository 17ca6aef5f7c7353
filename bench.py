#!/usr/bin/env python3
"""Benchmark of the hot path: Q4_K dequantize-GEMV 1 x 4096 -> 14336 on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Without --workload (or with gemv_q4k) it measures the headline configuration described
below.  The other workloads are the remaining baseline configurations and the ops around the
matmul, timed the same way (one JSON line each).

A step is one call of the quantized matmul (m = 1) over one weight matrix.  The weights
rotate over 16 distinct copies (504 MiB) so that no cache level can serve them: every step
streams its 33 MB from HBM.

Timing method (the same for every workload, whatever --steps and --warmup say):
  * warm-up: at least max(W, 200) steps AND at least 50 ms of device work;
  * then a region of exactly K steps is enqueued R times back to back on the stream the
    kernels run on, with one event between regions (R is at least 50 and grows until the
    regions cover about 100 ms); nothing synchronises inside that sequence;
  * `ms_per_step` is the MEDIAN over the R regions of (region time / K); p10 and p90 of the
    same set, R and the summed region time are printed beside it.
So `--steps 20 --warmup 5` and the defaults give the same figure.
"""
from __future__ import annotations

import argparse
import gc
import json
import math
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

WARMUP_MIN_STEPS = 200
WARMUP_MIN_SECONDS = 0.05
REGIONS_MIN = 50
REGIONS_MAX = 500
REGIONS_TARGET_SECONDS = 0.1
MAX_TIMED_STEPS = 400_000


# HBM bytes per launch of the timed kernel on the headline workload: not measured by this
# program (hardware counters need the profiler) but by two counter passes of this same command
# under rocprofv3 (FETCH_SIZE, then WRITE_SIZE, per dispatch), each scaled by what the same
# counter reads for a plain copy of known size; the summary sits in profiles/ beside the
# kernel trace.
TRAFFIC_BYTES_PER_LAUNCH = 33_374_000
TRAFFIC_SOURCE = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by a plain copy (profiles/)"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def percentile(sorted_vals, q):
    """Linear-interpolated percentile of an ascending list."""
    if len(sorted_vals) == 1:
        return sorted_vals[0]
    pos = q * (len(sorted_vals) - 1)
    lo = int(math.floor(pos))
    hi = min(lo + 1, len(sorted_vals) - 1)
    return sorted_vals[lo] + (sorted_vals[hi] - sorted_vals[lo]) * (pos - lo)


def parse_options(args):
    return {k: int(v) for k, v in (o.split("=", 1) for o in args.option)}


def measure(torch, enqueue_region, steps: int, warmup: int):
    """Times regions of exactly `steps` steps.  `enqueue_region(r)` enqueues the steps of region
    number r on torch's current stream (the stream the library launches on, so the events below
    see exactly those kernels) and returns without synchronising.

    Returns a dict: median / p10 / p90 microseconds per step, regions, timed seconds."""
    steps = max(1, steps)
    # warm-up floor: launches and device time, independent of the command line
    done, t0, r = 0, time.perf_counter(), 0
    torch.cuda.synchronize()
    while done < max(warmup, WARMUP_MIN_STEPS) or time.perf_counter() - t0 < WARMUP_MIN_SECONDS:
        enqueue_region(r)
        torch.cuda.synchronize()
        done += steps
        r += 1
    # one probe region sizes the number of repeats
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    enqueue_region(r)
    e1.record()
    torch.cuda.synchronize()
    r += 1
    region_s = max(e0.elapsed_time(e1) * 1e-3, 1e-7)
    regions = int(min(REGIONS_MAX, max(REGIONS_MIN, math.ceil(REGIONS_TARGET_SECONDS / region_s))))
    regions = max(10, min(regions, MAX_TIMED_STEPS // steps))
    events = [torch.cuda.Event(enable_timing=True) for _ in range(regions + 1)]
    # The launches are enqueued by host code that allocates Python objects; a pass of Python's
    # cyclic garbage collector in the middle of that (tens of ms with torch loaded) would starve
    # the GPU and be counted as kernel time.
    gc.collect()
    gc.disable()
    try:
        torch.cuda.synchronize()
        events[0].record()
        for i in range(regions):
            enqueue_region(r + i)
            events[i + 1].record()
        torch.cuda.synchronize()
    finally:
        gc.enable()
    per_step_us = sorted(events[i].elapsed_time(events[i + 1]) * 1e3 / steps for i in range(regions))
    return {"us": percentile(per_step_us, 0.5), "p10_us": percentile(per_step_us, 0.1),
            "p90_us": percentile(per_step_us, 0.9), "regions": regions,
            "timed_region_s": sum(per_step_us) * steps * 1e-6}


def timing_fields(t, steps, warmup):
    return {"steps": steps, "warmup": warmup, "ms_per_step": round(t["us"] / 1e3, 6), "us_per_call": round(t["us"], 3),
            "p10_us": round(t["p10_us"], 3), "p90_us": round(t["p90_us"], 3), "repeats": t["regions"],
            "timed_region_s": round(t["timed_region_s"], 4),
            "timing": "median over `repeats` back-to-back regions of `steps` calls each, events on the launching stream; "
                      "launch-to-launch gaps included",
            # what rocprofv3 reports as the kernel's own duration is not visible to events on the
            # stream; the committed kernel trace holds it
            "kernel_us": None}


BLOCK_BYTES = {8: 34, 12: 144, 13: 176, 14: 210}
TAGS = {8: "Q8_0", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K"}


def device_weight_any(torch, g, dtype: int, rows: int, k: int):
    """Random blocks of any of the four formats generated on the device (distributions of the
    baseline configurations: uniform quants, f16 d / dmin in (0.001, 0.05), Q6_K d in
    (0.001, 0.02) with int8 scales in -64..63)."""
    from gllm_amd.ggml import row_bytes
    w = torch.randint(0, 256, (rows * row_bytes(dtype, k),), dtype=torch.uint8, device="cuda", generator=g)
    b = w.view(-1, BLOCK_BYTES[dtype])
    nb = b.shape[0]
    if dtype in (12, 13):
        d = (torch.rand(nb, 2, device="cuda", generator=g) * 0.049 + 0.001).to(torch.float16)
        b[:, 0:4] = d.view(torch.uint8).view(-1, 4)
    elif dtype == 14:
        d = (torch.rand(nb, 1, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16)
        b[:, 208:210] = d.view(torch.uint8).view(-1, 2)
        b[:, 192:208] = ((b[:, 192:208] & 0x7F).to(torch.int16) - 64).to(torch.int8).view(torch.uint8)
    else:
        d = (torch.rand(nb, 1, device="cuda", generator=g) * 0.049 + 0.001).to(torch.float16)
        b[:, 0:2] = d.view(torch.uint8).view(-1, 2)
    return w


def cpu_time(fn, budget_s=8.0, max_reps=200):
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or reps >= max_reps:
            return dt / reps, reps, dt


def run_other(args):
    print(json.dumps(workload_result(args, args.workload, not args.no_cpu)), flush=True)


def workload_result(args, name, want_cpu):
    """The baseline configurations other than the headline one, and the ops on either side of the
    matmul.  Same timing method; weights (or outputs, for the write-dominated ops) rotate over
    enough copies to exceed the 256 MB Infinity Cache.  Returns the JSON line's dict."""
    import numpy as np
    import torch

    from gllm_amd.backend import HipBackend
    from gllm_amd.ggml import row_bytes
    from gllm_amd.synth import random_activations, random_gate_logits, random_weight
    from oracle import cref  # the checker, here only as the CPU baseline leg

    hip = HipBackend(0, options=parse_options(args))
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    threads = max(1, min(os.cpu_count() or 1, 16))
    steps = args.steps
    sec = sample = None
    extra = {}

    def rotating(run_one, copies):
        """Region r runs steps number r * steps .. of an endless rotation over `copies` inputs."""
        def region(r):
            base = r * steps
            for i in range(steps):
                run_one((base + i) % copies)
        return region

    if name in ("gemv_q4k_4096", "gemv_q6k", "gemm_m16", "gemm_m32", "gemm_m64", "layer_mix", "layer_mix_m4", "layer_mix_m32",
                "lm_head_q6k", "down_q6k", "down_q4k", "down_q6k_m2", "down_q4k_m4", "gemv_q8_0", "gemv_q5k", "qkv_q4k", "down_q5k"):
        if name.startswith("layer_mix"):
            mm = int(name.split("_m")[2]) if name.count("_m") == 2 else 1  # decode, or batched decode of 4 / 32 sequences
            ops = [(12, 6144, 4096, mm), (12, 4096, 4096, mm), (12, 2 * 14336, 4096, mm), (14, 4096, 14336, mm)]
            copies = 3
        else:
            dtype, n, k, m = {"gemv_q4k_4096": (12, 4096, 4096, 1), "gemv_q6k": (14, 14336, 4096, 1),
                              "gemv_q8_0": (8, 14336, 4096, 1), "gemv_q5k": (13, 14336, 4096, 1),
                              "gemm_m16": (12, 14336, 4096, 16), "gemm_m32": (12, 14336, 4096, 32),
                              "gemm_m64": (12, 14336, 4096, 64),
                              # the down projection of the layer: few weight rows (16 per CU), long rows
                              "down_q6k": (14, 4096, 14336, 1), "down_q4k": (12, 4096, 14336, 1), "down_q5k": (13, 4096, 14336, 1),
                              # the fused Q, K and V projection of the layer: 24 weight rows per CU
                              "qkv_q4k": (12, 6144, 4096, 1),
                              "down_q6k_m2": (14, 4096, 14336, 2), "down_q4k_m4": (12, 4096, 14336, 4),
                              # the output projection of a 128256-token vocabulary: Q6_K even in Q4 files
                              "lm_head_q6k": (14, 128256, 4096, 1)}[name]
            ops = [(dtype, n, k, m)]
            copies = max(2, (300 << 20) // (n * row_bytes(dtype, k)) + 1)
        sets = []
        for _ in range(copies):
            sets.append([(device_weight_any(torch, g, dt, n, k), torch.randn(m, k, device="cuda", generator=g),
                          torch.empty(m, n, device="cuda"), dt, m, n, k) for dt, n, k, m in ops])
        # one step = one call of the batch entry point over one set; a region is one C call over
        # `steps` consecutive sets of the rotation
        per_set = len(ops)
        # the matmuls of one set are independent of each other (their kernels may overlap); a set is
        # a step of its own and starts after the one before it
        batch = hip.make_batch([d for i in range(steps + copies) for d in sets[i % copies]],
                               after_previous=lambda i: i % per_set == 0)

        def region(r):
            hip.run_batch(batch, ((r * steps) % copies) * per_set, steps * per_set)
        byts = sum(n * row_bytes(dt, k) + m * k * 4 + m * n * 4 for dt, n, k, m in ops)
        flops = sum(2 * m * n * k for dt, n, k, m in ops)
        desc = " + ".join(f"{TAGS[dt]} M={m} K={k} N={n}" for dt, n, k, m in ops)
        t = measure(torch, region, steps, args.warmup)
        if want_cpu:
            # CPU: the oracle's reference-style path on the same shapes (bounded sample)
            host = [(random_weight(dt, n, k, seed=i), random_activations(m, k, seed=i), dt, m, n, k)
                    for i, (dt, n, k, m) in enumerate(ops)]
            sec, creps, cdt = cpu_time(lambda: [cref.quantized_matmul(w, x, dt, m, n, k, acc=cref.ACC_F32, threads=threads)
                                                for w, x, dt, m, n, k in host])
            sample = f"{creps} passes of the same shapes in {cdt:.1f} s"
    elif name == "moe":
        E, T, KK, H, F = 128, 16, 8, 4096, 1536
        gu = device_weight_any(torch, g, 12, E * 2 * F, H)
        dn = device_weight_any(torch, g, 14, E * H, F)
        x = torch.randn(T, H, device="cuda", generator=g)
        out = torch.empty(T, H, device="cuda")
        # The router is the library's: logits in, route table out, once per set of logits and
        # outside the timed region (routing is the gate's job, the metric is the expert matvec).
        # Capacity factor = number of experts: nothing is dropped (the default 1.25 gives
        # capacity 1 at 16 tokens over 128 experts and would drop most routes).
        tabs = []
        for s_ in range(8):
            logits = torch.from_numpy(random_gate_logits(T, E, seed=s_)).cuda()
            re_ = torch.empty(T, KK, dtype=torch.int32, device="cuda")
            rw = torch.empty(T, KK, device="cuda")
            rl = torch.empty(T, dtype=torch.int32, device="cuda")
            hip.moe_route(logits, KK, re_, rw, rl, capacity_factor=float(E))
            torch.cuda.synchronize()
            hit = len(np.unique(re_.cpu().numpy()))
            tabs.append((re_, rw, rl, hit))

        def run_one(i):
            re_, rw, rl, _ = tabs[i]
            hip.moe_matvec(gu, 12, dn, 14, x, out, H, F, E, re_, rw, rl)
        t = measure(torch, rotating(run_one, len(tabs)), steps, args.warmup)
        e_act = float(np.mean([tb[3] for tb in tabs]))
        byts = int(e_act * (2 * F * row_bytes(12, H) + H * row_bytes(14, F)) + 128 * H * 4 + 128 * F * 8 + T * H * 4)
        flops = 128 * 2 * (2 * F * H + H * F)
        desc = (f"MoE expert matvec: {E} experts, top-{KK}, {T} tokens, gate/up Q4_K [{2 * F}x{H}], down Q6_K [{H}x{F}], "
                f"{e_act:.1f} distinct experts hit per call on average, no capacity drop")
        if want_cpu:
            # CPU: 8 experts' worth of the same shapes (a sixteenth of the weights), 16 tokens top-2
            Ec = 8
            gu_h, dn_h = random_weight(12, Ec * 2 * F, H, seed=1), random_weight(14, Ec * H, F, seed=2)
            rc_ = cref.route(random_gate_logits(T, Ec, seed=0), 2, capacity_factor=float(Ec))
            xh = random_activations(T, H, seed=3)
            pairs_c = int(rc_["len"].sum())
            sec, creps, cdt = cpu_time(lambda: cref.moe_ffn(gu_h, 12, dn_h, 14, xh, H, F, Ec, rc_["expert"], rc_["weight"],
                                                            rc_["len"], acc=cref.ACC_F32, threads=threads))
            sec *= 128.0 / pairs_c  # the oracle works pair by pair: scale to the 128 pairs of the workload
            sample = (f"{creps} passes over {pairs_c} (token, expert) pairs of the same expert shapes in {cdt:.1f} s, "
                      f"scaled to 128 pairs")
    elif name in ("lm_head_argmax_q6k", "lm_head_then_argmax_q6k"):
        # the tail of a decode step: Q6_K lm_head over a 128256-token vocabulary and the greedy token;
        # as one call that never writes the logits, or as the matmul and Op::Argmax one after the other
        dtype, n, k = 14, 128256, 4096
        copies = 3
        fused = name == "lm_head_argmax_q6k"
        ws = [device_weight_any(torch, g, dtype, n, k) for _ in range(copies)]
        xs = [torch.randn(1, k, device="cuda", generator=g) for _ in range(copies)]
        logits = torch.empty(1, n, device="cuda")
        tok = torch.zeros(1, dtype=torch.int32, device="cuda")

        def run_one(i):
            if fused:
                hip.lm_head_argmax(ws[i], xs[i], dtype, n, k, tok)
            else:
                hip.quantized_matmul(ws[i], xs[i], logits, dtype, 1, n, k)
                hip.argmax(logits, tok)
        t = measure(torch, rotating(run_one, copies), steps, args.warmup)
        byts = n * row_bytes(dtype, k) + k * 4 + 4
        flops = 2 * n * k
        desc = (f"lm_head {TAGS[dtype]} 1x{k}->{n} + greedy token, " +
                ("one call, logits not written" if fused else "matmul then argmax") + f", rotating over {copies} matrices")
        if want_cpu:
            host_w, host_x = random_weight(dtype, n // 8, k, seed=0), random_activations(1, k, seed=0)
            sec, creps, cdt = cpu_time(lambda: cref.argmax_token(
                cref.quantized_matmul(host_w, host_x, dtype, 1, n // 8, k, acc=cref.ACC_F32, threads=threads)[0]))
            sec *= 8.0
            sample = f"{creps} passes over an eighth of the vocabulary ({n // 8} rows) in {cdt:.1f} s, scaled by 8"
    elif name.startswith("dequant_"):
        # Backend::dequantize of one 14336 x 4096 weight matrix: block bytes in, 4 bytes per element out
        dtype = {"dequant_q4k": 12, "dequant_q5k": 13, "dequant_q6k": 14, "dequant_q8_0": 8}.get(name)
        if dtype is None:
            log(f"bench.py: unknown workload {name}")
            sys.exit(2)
        n, k = 14336, 4096
        copies = 3
        ws = [device_weight_any(torch, g, dtype, n, k) for _ in range(copies)]
        outs = [torch.empty(n * k, device="cuda") for _ in range(copies)]
        t = measure(torch, rotating(lambda i: hip.dequantize(ws[i], outs[i], dtype), copies), steps, args.warmup)
        byts = n * row_bytes(dtype, k) + n * k * 4
        flops = 0
        desc = f"Backend::dequantize {TAGS[dtype]} {n} x {k} (block bytes in, f32 out), rotating over {copies} matrices"
        if want_cpu:
            host_w = random_weight(dtype, n // 8, k, seed=0)
            sec, creps, cdt = cpu_time(lambda: cref.dequantize(host_w, dtype))
            sec *= 8.0
            sample = f"{creps} decodes of an eighth of the matrix ({n // 8} x {k}) on one thread in {cdt:.1f} s, scaled by 8"
            threads = 1
    elif name in ("ffn_m1", "ffn_m4", "ffn_m32"):
        # dense feed-forward block of the layer mix: gate and up Q4_K 4096 -> 14336, SwiGLU, down Q6_K
        # 14336 -> 4096; algorithmic bytes = the three matrices once + x in + out (the intermediates
        # are the implementation's own traffic)
        mm = int(name.split("_m")[1])
        H, F = 4096, 14336
        copies = 3
        sets = []
        for _ in range(copies):
            gu = device_weight_any(torch, g, 12, 2 * F, H)
            half = gu.numel() // 2
            sets.append((gu[:half], gu[half:], device_weight_any(torch, g, 14, H, F),
                         torch.randn(mm, H, device="cuda", generator=g), torch.empty(mm, H, device="cuda")))

        def run_one(i):
            ga, up_, dn, xx, oo = sets[i]
            hip.ffn_swiglu(ga, up_, 12, dn, 14, xx, oo, mm, H, F)
        t = measure(torch, rotating(run_one, copies), steps, args.warmup)
        byts = 2 * F * row_bytes(12, H) + H * row_bytes(14, F) + 2 * mm * H * 4
        flops = 2 * mm * (2 * F * H + H * F)
        desc = f"dense FFN M={mm}: gate/up Q4_K {H}->{F}, SwiGLU, down Q6_K {F}->{H}, rotating over {copies} weight sets"
        if want_cpu:
            Fc = F // 8  # an eighth of the intermediate size: an eighth of every matrix
            hg, hu = random_weight(12, Fc, H, seed=1), random_weight(12, Fc, H, seed=2)
            hd = random_weight(14, H, Fc, seed=3)
            hx = random_activations(mm, H, seed=4)
            sec, creps, cdt = cpu_time(lambda: cref.ffn_swiglu(hg, hu, 12, hd, 14, hx, mm, H, Fc, acc=cref.ACC_F32, threads=threads))
            sec *= 8.0
            sample = f"{creps} passes at an eighth of the intermediate size ({Fc}) in {cdt:.1f} s, scaled by 8"
    elif name.startswith("gather_"):
        # Op::QuantGather: 2048 token ids (a prefill) into a 32000 x 4096 embedding table;
        # algorithmic bytes = the looked-up rows' block bytes + the ids in, 4 bytes per element out
        dtype = {"gather_q4k": 12, "gather_q6k": 14, "gather_q8_0": 8}.get(name)
        if dtype is None:
            log(f"bench.py: unknown workload {name}")
            sys.exit(2)
        vocab, hidden, count = 32000, 4096, 2048
        table = device_weight_any(torch, g, dtype, vocab, hidden)
        copies = 12  # 12 x 33.5 MB of outputs rotate past the Infinity Cache
        ids = [torch.randint(0, vocab, (count,), generator=g, device="cuda", dtype=torch.int32) for _ in range(copies)]
        outs = [torch.empty(count * hidden, device="cuda") for _ in range(copies)]
        t = measure(torch, rotating(lambda i: hip.quant_gather(table, dtype, vocab, hidden, ids[i], outs[i]), copies),
                    steps, args.warmup)
        byts = count * row_bytes(dtype, hidden) + count * 4 + count * hidden * 4
        flops = 0
        desc = (f"Op::QuantGather {TAGS[dtype]}: {count} ids into a {vocab} x {hidden} table (row blocks in, f32 rows out), "
                f"rotating over {copies} id sets and outputs")
        if want_cpu:
            host_t = random_weight(dtype, 1024, hidden, seed=0)
            host_ids = np.random.default_rng(0).integers(0, 1024, count // 8).astype(np.uint32)
            sec, creps, cdt = cpu_time(lambda: cref.quant_gather(host_t, dtype, 1024, hidden, host_ids))
            sec *= 8.0
            sample = f"{creps} lookups of {count // 8} ids in a 1024-row table on one thread in {cdt:.1f} s, scaled by 8"
            threads = 1
    else:
        log(f"bench.py: unknown workload {name}")
        sys.exit(2)

    us = t["us"]
    gbs = byts / us / 1e3
    result = {
        "metric": f"{name}: achieved HBM GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        **timing_fields(t, steps, args.warmup),
        "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 2), "tflops": round(flops / us / 1e6, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if name.startswith("gemm") else ("f32" if name.startswith(("dequant", "gather")) else "i8"), "data": "synthetic",
        "config": {"workload": desc, "bytes_per_call": byts, **extra, **({"options": parse_options(args)} if args.option else {})},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
    }
    if sec is not None:
        result["cpu_baseline"] = {"value": round(byts / sec / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
                                  "us_per_call": round(sec * 1e6, 1), "sample": sample}
    result["config"]["kernel"] = hip.last_kernel_name()
    log(f"{name}: {us:.2f} us/call (p10 {t['p10_us']:.2f}, p90 {t['p90_us']:.2f}, {t['regions']} regions of {steps}), "
        f"{gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS * 100:.1f}% of 8 TB/s)")
    return result


# The baseline's configurations beside the headline one: timed in the default run as well (GPU legs
# only), so that every figure quoted for them is one a plain `python bench.py` prints.
CONTEXT_CONFIGS = (("cfg1_gemv_q4k_4096", "gemv_q4k_4096"), ("cfg2_gemv_q6k", "gemv_q6k"), ("cfg3_layer_mix", "layer_mix"),
                   ("cfg4_gemm_m16", "gemm_m16"), ("cfg4_gemm_m32", "gemm_m32"), ("cfg4_gemm_m64", "gemm_m64"), ("cfg5_moe", "moe"))


def context_configs(args, torch):
    out = {}
    for key, name in CONTEXT_CONFIGS:
        r = workload_result(args, name, False)
        out[key] = {"workload": name, "us_per_call": r["us_per_call"], "p10_us": r["p10_us"], "p90_us": r["p90_us"],
                    "gbs": r["value"], "frac": r["roofline"]["frac"], "tflops": r["tflops"],
                    "bytes_per_call": r["config"]["bytes_per_call"], "kernel": r["config"]["kernel"], "what": r["config"]["workload"]}
        gc.collect()
        torch.cuda.empty_cache()
    return out


def launch_cadence_us(torch, kernels: int = 500):
    """Time per kernel of a captured sequence of empty-handed kernels on one stream (each adds 1 to
    one float): what the device needs from one dependent launch to the next, whatever the kernel."""
    t = torch.zeros(1, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            t.add_(1.0)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(kernels):
                t.add_(1.0)
        e = [torch.cuda.Event(enable_timing=True) for _ in range(12)]
        graph.replay()
        side.synchronize()
        for i in range(11):
            e[i].record(side)
            graph.replay()
        e[11].record(side)
        side.synchronize()
    per = sorted(e[i].elapsed_time(e[i + 1]) * 1e3 / kernels for i in range(11))
    return round(per[len(per) // 2], 3)


def cpu_baseline(budget_s: float = 12.0, simd_budget_s: float = 5.0):
    """The oracle's reference-faithful matmul (scalar per-block decode, f32 multiply-add: what the
    reference ships for K-quants) on the host cores, on the same shape with the same generator,
    repeated for about `budget_s` seconds; beside it the oracle's vectorised flavours (AVX2, and
    AVX-512 where the host has it: block decode and f32 sums in vector registers) for
    `simd_budget_s` seconds each."""
    from gllm_amd.ggml import row_bytes
    from gllm_amd.synth import random_activations, random_weight
    from oracle import cref
    threads = max(1, min(os.cpu_count() or 1, 16))
    w = random_weight(DTYPE, N, K_DIM, seed=0)
    x = random_activations(M, K_DIM, seed=0)
    bytes_per_call = N * row_bytes(DTYPE, K_DIM) + M * K_DIM * 4 + M * N * 4

    def leg(fn, budget):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget or reps >= 20000:
                return reps, dt

    reps, dt = leg(lambda: cref.quantized_matmul(w, x, DTYPE, M, N, K_DIM, acc=cref.ACC_F32, threads=threads), budget_s)
    out = {"value": round(bytes_per_call * reps / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
           "us_per_call": round(dt / reps * 1e6, 1),
           "sample": f"{reps} calls of the same 1x{K_DIM}x{N} Q4_K matmul (C restatement of the reference's "
                     f"scalar decode + f32 FMA, rows split over {threads} threads) in {dt:.1f} s"}
    for tag, have, fn in (("avx2", cref.have_avx2, cref.quantized_matmul_avx2),
                          ("avx512", getattr(cref, "have_avx512", lambda: False), getattr(cref, "quantized_matmul_avx512", None))):
        if fn is None or not have():
            continue
        reps, dt = leg(lambda: fn(w, x, DTYPE, M, N, K_DIM, threads=threads), simd_budget_s)
        out[tag] = {"value": round(bytes_per_call * reps / dt / 1e9, 3), "unit": "GB/s", "cores": threads,
                    "us_per_call": round(dt / reps * 1e6, 1),
                    "sample": f"{reps} calls of the same matmul with the oracle's {tag.upper()} decode and vector f32 sums "
                              f"over {threads} threads in {dt:.1f} s"}
    return out


def main():
    global COPIES
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-context", action="store_true",
                    help="skip the cache-resident and copy-rate context runs (profiling: only the timed kernel launches)")
    ap.add_argument("--workload", default="gemv_q4k",
                    help="gemv_q4k (headline, default), gemv_q4k_4096, gemv_q5k, gemv_q6k, gemv_q8_0, layer_mix, layer_mix_m4, layer_mix_m32, gemm_m16, gemm_m32, gemm_m64, qkv_q4k, down_q6k, down_q4k, down_q5k, down_q6k_m2, down_q4k_m4, lm_head_q6k, lm_head_argmax_q6k, lm_head_then_argmax_q6k, ffn_m1, ffn_m4, ffn_m32, moe, "
                         "dequant_q4k, dequant_q5k, dequant_q6k, dequant_q8_0, gather_q4k, gather_q6k, gather_q8_0")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="kernel-family option of the library for this run (repeatable), e.g. mm8s=0")
    ap.add_argument("--no-configs", action="store_true", help="skip the other baseline configurations in the headline run's context")
    ap.add_argument("--copies", type=int, default=COPIES,
                    help="weight copies the headline workload rotates over (default 16 = 504 MiB, past every cache; fewer "
                         "shows what the caches give: 2 copies fit the memory-side cache but no L2)")
    ap.add_argument("--real-chain", action="store_true", help="every matmul reads the first K outputs of the one before it")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch plain device-to-device copies of one 33 MB weight buffer (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build measures one GPU; the quantized matmul path has no multi-GPU part "
            "(rows would shard by N with no collective). Run with --gpus 1.")
        sys.exit(2)
    if args.steps < 1:
        log("bench.py: --steps must be at least 1")
        sys.exit(2)

    import torch

    from gllm_amd.backend import HipBackend
    from gllm_amd.ggml import row_bytes

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    if args.workload != "gemv_q4k":
        run_other(args)
        return
    hip = HipBackend(0, options=parse_options(args))
    COPIES = max(1, args.copies)  # (module-level name: the helpers below read it)
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    ws = [device_weight_any(torch, g, DTYPE, N, K_DIM) for _ in range(COPIES)]
    g.manual_seed(1)
    x = torch.randn(M, K_DIM, device="cuda", generator=g)
    ys = [torch.empty(M, N, device="cuda") for _ in range(COPIES)]
    nb = ws[0].numel()
    bytes_per_call = N * row_bytes(DTYPE, K_DIM) + M * K_DIM * 4 + M * N * 4  # 33,103,872
    steps = args.steps

    # One list of steps + COPIES descriptors; region r is one C call over `steps` consecutive
    # entries starting where region r - 1 stopped in the rotation.
    # every entry is a call of its own: it starts after the one before it has finished
    if args.real_chain:
        ys = [torch.zeros(M, N, device="cuda") for _ in range(steps + COPIES)]
        rotating = hip.make_batch([(ws[i % COPIES], x if i == 0 else ys[i - 1], ys[i], DTYPE, M, N, K_DIM) for i in range(steps + COPIES)],
                                  after_previous=lambda i: True)
    else:
        rotating = hip.make_batch([(ws[i % COPIES], x, ys[i % COPIES], DTYPE, M, N, K_DIM) for i in range(steps + COPIES)],
                                  after_previous=lambda i: True)
    resident = hip.make_batch([(ws[0], x, ys[0], DTYPE, M, N, K_DIM)] * steps, after_previous=lambda i: True)

    if args.copy_probe:
        # A plain copy kernel of known size: 33,030,144 bytes read and as many written per launch.
        dst = torch.empty_like(ws[0])
        for i in range(8):
            dst.copy_(ws[i % COPIES])
        torch.cuda.synchronize()

    t = measure(torch, lambda r: hip.run_batch(rotating, (r * steps) % COPIES, steps), steps, args.warmup)
    main_kernel = hip.last_kernel_name()
    us_per_call = t["us"]
    gbs = bytes_per_call / (us_per_call * 1e-6) / 1e9

    # context figures: cache-resident weights, and the rate of a plain device-to-device copy
    context = None
    if not args.no_context:
        t1 = measure(torch, lambda r: hip.run_batch(resident, 0, steps), steps, args.warmup)
        dsts = [torch.empty_like(ws[0]) for _ in range(4)]
        tc = measure(torch, lambda r: [dsts[i % 4].copy_(ws[(r * 20 + i) % COPIES]) for i in range(20)], 20, 20)
        # the same matmuls as independent entries of the batch (no entry waits for the one before
        # it): the library runs them as one launch whose weight stream never stops between entries
        free = hip.make_batch([(ws[i % COPIES], x, ys[i % COPIES], DTYPE, M, N, K_DIM) for i in range(steps + COPIES)])
        t2 = measure(torch, lambda r: hip.run_batch(free, (r * steps) % COPIES, steps), steps, args.warmup)
        free_kernel = hip.last_kernel_name()
        # (those entries share one activation row, as the Q, K and V projections of a token do, and
        # a workgroup of the chained launch prepares a shared row once; with a row of its own per
        # entry every entry is prepared)
        xs = [torch.randn(M, K_DIM, device="cuda", generator=g) for _ in range(COPIES)]
        own = hip.make_batch([(ws[i % COPIES], xs[i % COPIES], ys[i % COPIES], DTYPE, M, N, K_DIM) for i in range(steps + COPIES)])
        t3 = measure(torch, lambda r: hip.run_batch(own, (r * steps) % COPIES, steps), steps, args.warmup)
        context = {"launch_cadence_us": launch_cadence_us(torch),
                   "cache_resident_us_per_call": round(t1["us"], 3),
                   "device_copy_gbs_read_plus_write": round(2 * nb / tc["us"] / 1e3, 1),
                   "independent_entries": {"us_per_call": round(t2["us"], 3), "p10_us": round(t2["p10_us"], 3),
                                           "p90_us": round(t2["p90_us"], 3),
                                           "gbs": round(bytes_per_call / (t2["us"] * 1e-6) / 1e9, 1),
                                           "frac": round(bytes_per_call / (t2["us"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                           "kernel": free_kernel, "activations": "one row shared by all entries",
                                           "own_row_per_entry_us_per_call": round(t3["us"], 3),
                                           "own_row_per_entry_frac": round(bytes_per_call / (t3["us"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}}
    log(f"Q4_K GEMV 1x{K_DIM}x{N}: {us_per_call:.2f} us/call (p10 {t['p10_us']:.2f}, p90 {t['p90_us']:.2f}; "
        f"{t['regions']} regions of {steps} calls), {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS * 100:.1f}% of 8 TB/s), "
        f"{2 * N * K_DIM / (us_per_call * 1e-6) / 1e12:.2f} TFLOP/s")
    if context:
        log(f"  same weights every call (cache resident): {context['cache_resident_us_per_call']:.2f} us/call")
        ie = context["independent_entries"]
        log(f"  as independent entries of one batch call ({ie['kernel']}): {ie['us_per_call']:.2f} us/call, "
            f"{ie['gbs']:.0f} GB/s ({ie['frac'] * 100:.1f}% of 8 TB/s); with an activation row of its own per entry "
            f"{ie['own_row_per_entry_us_per_call']:.2f} us/call ({ie['own_row_per_entry_frac'] * 100:.1f}%)")
        log(f"  plain device-to-device copy of the same 33 MB buffers: {context['device_copy_gbs_read_plus_write']:.0f} GB/s read+write")
        log(f"  one dependent launch to the next, whatever the kernel (graph of one-float kernels): {context['launch_cadence_us']:.2f} us")

    result = {
        "metric": "Q4_K GEMV 1x4096x14336: achieved HBM GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        **timing_fields(t, steps, args.warmup),
        "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 2),
        "target_pct_of_hbm_peak": 70.0,
        "tflops": round(2 * N * K_DIM / (us_per_call * 1e-6) / 1e12, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {**({"options": parse_options(args)} if args.option else {}),
                   "workload": f"Q4_K dequant-GEMV M=1 K={K_DIM} N={N} (GGUF 144-byte super-blocks), f32 activations "
                               f"~N(0,1) as 23-bit block fixed point, int8 MFMA with i32 accumulation, f32 scales; "
                               f"weights rotate over {COPIES} copies ({COPIES * nb >> 20} MiB) so every call reads HBM",
                   "bytes_per_call": bytes_per_call, "kernel": main_kernel},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": TRAFFIC_SOURCE,
                     "note": "achieved = 33,103,872 algorithmic bytes / median event time per call; "
                             "the event time includes the gap between back-to-back launches"},
    }
    if context:
        del ws, ys, rotating, resident, free, own, xs, dsts
        gc.collect()
        torch.cuda.empty_cache()
        if not args.no_configs:
            context["configs"] = context_configs(args, torch)
        result["context"] = context
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
        log(f"  CPU baseline: {result['cpu_baseline']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
