#!/usr/bin/env python3
"""Decode-step self-attention benchmark (one MI355X).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3]

One step = one pass of the hot path (RoPE -> KV append -> masked attention over the cache) for a
whole batch, through the C ABI, on synthetic seeded inputs already resident in HBM.  Prints ONE
JSON line.  `value` is algorithmic bytes per step / time per step (GB/s); `ms_per_step` carries the
latency half of the metric.  `roofline` prices the streaming kernel alone (HIP events around
back-to-back launches of that pass); `cpu_baseline` is the scalar CPU oracle timed on this
machine's host cores on a bounded sample of the same workload.
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

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak

# name -> (B, H, D, ctx, L, dtype, extras)
WORKLOADS = {
    "cfg1": dict(B=1, H=4, D=64, ctx=128, L=128, dtype="f32", copies=64),
    "cfg2": dict(B=8, H=32, D=128, ctx=1024, L=1024, dtype="f16", copies=6),
    "cfg3": dict(B=64, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=1),
    "cfg4": dict(B=1, H=32, D=128, ctx=4096, L=4096, dtype="f16", copies=12),
    "cfg5": dict(B=32, H=40, D=128, ctx=None, L=4096, dtype="f16", copies=1, ragged=True),
    # exploration shapes (not among the five headline configurations)
    "x13b_uniform": dict(B=32, H=40, D=128, ctx=4096, L=4096, dtype="f16", copies=1),
    "x7b_halffull": dict(B=64, H=32, D=128, ctx=2048, L=4096, dtype="f16", copies=1),
    "x7b_f32": dict(B=64, H=32, D=128, ctx=2048, L=2048, dtype="f32", copies=1),  # the reference's cache type
    "xb80": dict(B=80, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=1),
    "xb48": dict(B=48, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=1),
    "xb100": dict(B=100, H=32, D=128, ctx=1024, L=1024, dtype="f16", copies=1),
    "xb32": dict(B=32, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=1),
    "xb16": dict(B=16, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=1),
    "xb4": dict(B=4, H=32, D=128, ctx=2048, L=2048, dtype="f16", copies=4),
    "xb1_c1024": dict(B=1, H=32, D=128, ctx=1024, L=4096, dtype="f16", copies=12),  # cfg4 with a quarter / half of
    "xb1_c2048": dict(B=1, H=32, D=128, ctx=2048, L=4096, dtype="f16", copies=12),  # the context: fixed vs per-byte cost
    "xd64": dict(B=64, H=64, D=64, ctx=2048, L=2048, dtype="f16", copies=1),
    "xd256": dict(B=64, H=16, D=256, ctx=2048, L=2048, dtype="f16", copies=1),
}
HEADLINE = "cfg3"

# prompt-phase (seq_len > 1) shapes: a different roofline (FP32 MFMA), reported in TFLOP/s
PREFILL_WORKLOADS = {
    "prefill_7b_b8_s1024": dict(B=8, H=32, D=128, S=1024, P=0, L=1024, dtype="f16"),
    "prefill_7b_b8_s1024_f32": dict(B=8, H=32, D=128, S=1024, P=0, L=1024, dtype="f32"),
    "prefill_7b_b1_s4096": dict(B=1, H=32, D=128, S=4096, P=0, L=4096, dtype="f16"),
    "prefill_7b_b32_s128": dict(B=32, H=32, D=128, S=128, P=0, L=256, dtype="f16"),
}
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X published dense FP32 matrix rate (FP32 caches)
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 matrix rate (fp16 caches)


def bench_prefill(args) -> int:
    """Prints the JSON line of one prompt-phase workload."""
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    print(json.dumps(measure_prefill(args, args.workload, min(args.steps, 50), min(args.warmup, 5), args.repeats,
                                     cpu=not args.no_cpu)), flush=True)
    return 0


def measure_prefill(args, workload, steps, warm, repeats, cpu=False) -> dict:
    """One step = RoPE + append + dense attention of S new tokens per sequence (prompt phase).  Returns the
    workload's JSON object."""
    import numpy as np
    import torch

    from fasterllama_amd import capi, synth
    from fasterllama_amd.decode_attn import PrefillAttention

    capi.load()
    dev = torch.device("cuda:0")
    w = PREFILL_WORKLOADS[workload]
    B, H, D, S, P, L = w["B"], w["H"], w["D"], w["S"], w["P"], w["L"]
    np_dt = np.float16 if w["dtype"] == "f16" else np.float32
    t_dt = torch.float16 if w["dtype"] == "f16" else torch.float32
    q_h = synth.normal((B, S, H, D), np_dt, synth.TENSOR_Q, args.seed)
    k_h = synth.normal((B, S, H, D), np_dt, synth.TENSOR_K_NEW, args.seed)
    v_h = synth.normal((B, S, H, D), np_dt, synth.TENSOR_V_NEW, args.seed)
    freq_h = synth.freq_cis_table(L, D)
    # causal additive mask: masked entries hold -FLT_MAX as in the reference's driver
    # (samples/llama_fp16.cu:73-81), or -1e5 as in its kernel harness (samples/test.cu:427-437)
    masked = -1e5 if args.prefill_mask == "causal-1e5" else -float(np.finfo(np.float32).max)
    blk = 128 if args.prefill_mask == "block-causal" else 1  # block-causal: whole 128-token blocks see each other
    mask_h = np.where(np.arange(L)[None, :] // blk > np.arange(L)[:, None] // blk, masked, 0.0).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    q, k, v, freq, mask = t(q_h), t(k_h), t(v_h), t(freq_h), t(mask_h)
    kc = torch.zeros(B, H, L, D, dtype=t_dt, device=dev)
    vc = torch.zeros_like(kc)
    out = torch.empty(B, H, S, D, dtype=torch.float32, device=dev)
    op = PrefillAttention(B, H, D, L, S, t_dt, device=dev, fast_qk=args.prefill_fast_qk)
    # the reference installs ONE mask for every layer and call (samples/llama_fp16.cu:139-150): its tile classes are
    # computed once, outside the timed step (fl_prefill_mask_classify), unless --prefill-classify-per-call
    table = None
    if args.prefill_mask != "none" and not args.prefill_classify_per_call:
        table = op.classify_mask(mask)
    extra = {}
    if args.segment == "int32-int8":
        # the segment as OpenDecoder::forward feeds it: int32 accumulators + scales in, per-token INT8 + scale out, no
        # float output (the float result passes through the workspace to the quantisation kernel)
        cpu = False
        rng = np.random.default_rng(args.seed)
        q, k, v = (torch.from_numpy(rng.integers(-20000, 20000, (B, S, H, D), dtype=np.int32)).to(dev) for _ in range(3))
        extra = dict(
            qkv_inp_scale=torch.from_numpy(((rng.random(B * S) + 0.5) * 2e-3).astype(np.float32)).to(dev),
            q_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            k_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            v_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            out_int8=torch.empty(B, S, H * D, dtype=torch.int8, device=dev),
            out_scale=torch.empty(B, S, dtype=torch.float32, device=dev))
        out = None
    io = op.make_io(q, k, v, kc, vc, freq, out, start_pos=P, attn_mask=None if args.prefill_mask == "none" else mask,
                    mask_tile_classes=table, **extra)
    stream = torch.cuda.current_stream(dev)

    def run(n):
        for _ in range(n):
            st = op.launch_prefill(io, S, stream)
            if st != 0:
                raise capi.FlAttnError(st, capi.strerror(st))

    run(warm)
    torch.cuda.synchronize()
    ms, ms_all = time_region(torch, stream, run, steps, repeats)

    # the attention kernel alone (fl_prefill_attn_forward_passes, pass 2: the cache rows are in place from the steps above)
    def run_attn(n):
        for _ in range(n):
            st = op.launch_prefill(io, S, stream, passes=2)
            if st != 0:
                raise capi.FlAttnError(st, capi.strerror(st))

    ms_attn, ms_attn_all = time_region(torch, stream, run_attn, steps, repeats)
    dense_flops = 4.0 * B * H * S * (P + S) * D  # every query against every key
    # FLOPs the kernels execute: 32x32 tiles whose mask entries are all <= -1e30 are dropped (their weights
    # are exactly 0); every other tile is multiplied.
    flops = dense_flops
    if args.prefill_mask != "none":
        rows = mask_h[P:P + S, :P + S]
        pad_q, pad_k = (-S) % 32, (-(P + S)) % 32
        tiles = np.pad(rows, ((0, pad_q), (0, pad_k)), constant_values=-np.inf)
        tiles = tiles.reshape(tiles.shape[0] // 32, 32, tiles.shape[1] // 32, 32)
        open_tiles = int(((tiles > -1e30) | np.isnan(tiles)).any(axis=(1, 3)).sum())
        flops = 4.0 * B * H * open_tiles * 32 * 32 * D
    tflops = flops / (ms * 1e-3) / 1e12
    tflops_attn = flops / (ms_attn * 1e-3) / 1e12
    peak = MFMA_FP16_PEAK_TFLOPS if w["dtype"] == "f16" else MFMA_FP32_PEAK_TFLOPS

    max_err = None
    cpu_leg = None
    if cpu:
        from oracle import ref  # checker / baseline only
        nb = 1
        kc_s = np.zeros((nb, H, L, D), np_dt)
        vc_s = np.zeros_like(kc_s)
        nthreads = max(1, min(16, os.cpu_count() or 1))
        t1 = time.perf_counter()
        want = ref.prefill_attn(q_h[:nb], k_h[:nb], v_h[:nb], kc_s, vc_s, freq_h, start_pos=P,
                                attn_mask=None if args.prefill_mask == "none" else mask_h, threads=nthreads)
        dt_cpu = time.perf_counter() - t1
        max_err = float(np.abs(out[:nb].cpu().numpy() - want).max())
        cpu_leg = {"value": round(4.0 * nb * H * S * (P + S) * D / dt_cpu / 1e12, 5), "unit": "TFLOP/s (dense count)", "cores": nthreads,
               "kind": "port", "sample": f"first {nb} of {B} sequences, scalar oracle with OpenMP over heads, {dt_cpu:.2f} s",
               "gpu_vs_oracle_max_abs_err": max_err}
    del kc, vc, q, k, v, out, io, op
    torch.cuda.empty_cache()
    return {
        "metric": f"prompt-phase attention TFLOP/s, {workload}", "value": round(tflops, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": steps, "warmup": warm, "repeats": repeats, "ms_per_step": round(ms, 5),
        "ms_per_step_all_regions": [round(x, 5) for x in ms_all], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 MFMA, f32 accumulate (f16 storage)" if w["dtype"] == "f16" else "f32 MFMA",
        "data": "synthetic (seeded splitmix64 + Box-Muller N(0,1), seed %d)" % args.seed,
        "config": {"workload": f"{workload}: B={B} H={H} D={D} S={S} start_pos={P} L={L} {w['dtype']} KV cache, "
                               + {"causal": "causal additive mask, -FLT_MAX above the diagonal",
                                  "causal-1e5": "causal additive mask, -1e5 above the diagonal",
                                  "block-causal": "additive mask, causal over blocks of 128 tokens, -FLT_MAX above",
                                  "none": "no mask"}[args.prefill_mask]
                               + (", fast first product (fp16 queries)" if args.prefill_fast_qk and w["dtype"] == "f16" else "")
                               + (", mask tiles classified once per mask" if table is not None else "")
                               + (", int32 accumulators in, INT8 + scale out" if args.segment == "int32-int8" else ""),
                   "flops_per_step": flops, "dense_flops_per_step": dense_flops,
                   "dense_tflops": round(dense_flops / (ms * 1e-3) / 1e12, 2),
                   "tokens_per_s": round(B * S / (ms * 1e-3), 1)},
        # the dominant kernel: the attention kernel alone, timed in a region of its own (pass 2 of the step)
        "roofline": {"bound": "mfma", "achieved": round(tflops_attn, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(tflops_attn / peak, 4), "traffic": None,
                     "kernel": "prefill_attn_f16_kernel" if w["dtype"] == "f16" and D <= 128 else
                               ("prefill_attn_kernel" if D <= 128 else "prefill_attn_wide_kernel"),
                     "kernel_us": round(ms_attn * 1e3, 2), "kernel_us_all_regions": [round(x * 1e3, 2) for x in ms_attn_all],
                     "step_frac": round(tflops / peak, 4)},
        "cpu_baseline": cpu_leg}


def prefill_summary(line):
    """The figures of one prompt-phase workload as they appear under other_configs."""
    return {"workload": line["config"]["workload"], "ms_per_step": line["ms_per_step"],
            "tflops_executed": line["value"], "tflops_dense_count": line["config"]["dense_tflops"],
            "mfma_peak_tflops": line["roofline"]["peak"], "frac_of_mfma_peak": line["roofline"]["step_frac"],
            "attention_kernel_us": line["roofline"]["kernel_us"], "attention_kernel_tflops_executed": line["roofline"]["achieved"],
            "attention_kernel_frac_of_mfma_peak": line["roofline"]["frac"],
            "note": "ms_per_step, tflops_* and frac_of_mfma_peak: whole step = append kernel + attention kernel; attention_kernel_*: "
                    "the attention kernel alone, timed in a region of its own; executed = tiles the causal mask leaves (-FLT_MAX "
                    "tiles are exact zeros and dropped), dense = every query against every key",
            "ms_per_step_all_regions": line["ms_per_step_all_regions"]}


def opendecoder_loop(B, H, D, L, P, layers, steps):
    """OpenDecoder::forward in the reference driver's layer loop (initialize(param[layer], buf) before every
    forward), timed by the C++ program fasterllama_amd/lib/open_decoder_bench; its JSON object, or an error note."""
    import subprocess

    from fasterllama_amd import build
    exe = build.outputs("cxxbench")
    if not os.path.exists(exe):
        return {"error": f"{exe} has not been built (python -m fasterllama_amd.build cxxbench)"}
    res = subprocess.run([exe] + [str(x) for x in (B, H, D, L, P, layers, steps)], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=300)
    if res.returncode != 0:
        return {"error": f"open_decoder_bench exited with {res.returncode}: {res.stderr.strip()[-300:]}"}
    return json.loads(res.stdout.strip().splitlines()[-1])

def measured_traffic(workload: str, mask: str):
    """HBM bytes per launch of the streaming kernel for this workload, as measured with rocprofv3 --pmc
    (FETCH_SIZE and WRITE_SIZE runs, scaled by what the same counters read for a copy kernel of known
    size) and recorded in profiles/hbm_traffic_per_launch.md; (None, None) when no row matches."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.md")
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 3 and cells[0] == workload and cells[1] == mask and cells[2].isdigit():
                    return int(cells[2]), "profiles/hbm_traffic_per_launch.md"
    except OSError:
        pass
    return None, None


def algorithmic_bytes(B, H, D, e, sum_ctx, has_mask=False, mean_ctx=0):
    """Bytes one step must move: K and V rows once, the token's q/k/v in, the two new rows out,
    the fp32 output, one RoPE row (and one mask row when a mask is given)."""
    kv = 2 * H * D * e * sum_ctx              # sum over sequences of ctx_b rows of K and of V
    tok = 3 * B * H * D * e + 2 * B * H * D * e
    out = B * H * D * 4
    small = D * 4 + (int(mean_ctx) * 4 if has_mask else 0)
    return kv + tok + out + small


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def time_region(torch, stream, run, steps, repeats):
    """ms per step of `run(steps)` between two events on `stream`: the median of `repeats` timed regions
    (and every region's figure)."""
    per_step = []
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        run(steps)
        e1.record(stream)
        torch.cuda.synchronize()
        per_step.append(e0.elapsed_time(e1) / steps)
    return median(per_step), per_step


def measure_decode(name, args, steps, warmup, repeats, mask="none", graph_steps=0, cpu=False, two_launches=False,
                   segment="attention", nsplit=0):
    """One decode workload: inputs to HBM, timed regions of the whole step and of the streaming kernel
    alone, optionally the HIP-graph replay and the CPU baseline.  Returns a dict of plain numbers."""
    import numpy as np
    import torch

    from fasterllama_amd import capi, synth
    from fasterllama_amd.decode_attn import DecodeAttention

    dev = torch.device("cuda:0")
    w = WORKLOADS[name]
    B, H, D, L = w["B"], w["H"], w["D"], w["L"]
    np_dt = np.float16 if w["dtype"] == "f16" else np.float32
    t_dt = torch.float16 if w["dtype"] == "f16" else torch.float32
    e = 2 if w["dtype"] == "f16" else 4
    ragged = bool(w.get("ragged"))
    copies = w["copies"]

    if ragged:
        lens = synth.uniform_int(B, 1, L, synth.TENSOR_LENS, args.seed)
        pos_h = (lens - 1).astype(np.int32)
        sum_ctx, max_ctx = int(lens.sum()), int(lens.max())
    else:
        lens = np.full(B, w["ctx"], np.int32)
        pos_h = None
        sum_ctx, max_ctx = B * w["ctx"], w["ctx"]
    start_pos = max_ctx - 1

    # ---- inputs: generated on the host by the seeded generator, then copied to HBM once
    t0 = time.time()
    q_h = synth.normal((B, 1, H, D), np_dt, synth.TENSOR_Q, args.seed)
    k_h = synth.normal((B, 1, H, D), np_dt, synth.TENSOR_K_NEW, args.seed)
    v_h = synth.normal((B, 1, H, D), np_dt, synth.TENSOR_V_NEW, args.seed)
    kc_h = synth.normal((B, H, L, D), np_dt, synth.TENSOR_K_CACHE, args.seed)
    vc_h = synth.normal((B, H, L, D), np_dt, synth.TENSOR_V_CACHE, args.seed)
    if ragged:  # rows the step must never read
        for b in range(B):
            kc_h[b, :, lens[b]:, :] = np.nan
            vc_h[b, :, lens[b]:, :] = np.nan
    freq_h = synth.freq_cis_table(L, D)
    q, k, v = (torch.from_numpy(a).to(dev) for a in (q_h, k_h, v_h))
    freq = torch.from_numpy(freq_h).to(dev)
    mask_h = None
    if mask != "none":
        fmax = float(np.finfo(np.float32).max)
        r, c = np.arange(L)[:, None], np.arange(L)[None, :]
        mask_h = np.where(c <= r if mask == "causal" else c < r, 0.0, -fmax).astype(np.float32)
    mask_d = None if mask_h is None else torch.from_numpy(mask_h).to(dev)
    pos_d = torch.from_numpy(pos_h).to(dev) if ragged else None
    # small workloads rotate over several cache copies so the rows do not sit in the 256 MB MALL
    caches = [(torch.from_numpy(kc_h).to(dev), torch.from_numpy(vc_h).to(dev)) for _ in range(copies)]
    out = torch.empty(B, H * D, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    gen_s = time.time() - t0

    op = DecodeAttention(B, H, D, L, t_dt, nsplit=nsplit, device=dev)
    if not two_launches:
        op.init_workspace()  # a split context is merged inside the streaming kernel: one launch per step
    plan = op.plan(max_ctx, ragged)
    extra = {}
    if segment == "int32-int8":
        # the segment as OpenDecoder::forward feeds it: int32 accumulators of the INT8 projections with
        # activation/weight scales in, quantised attention output out
        rng = np.random.default_rng(args.seed)
        q, k, v = (torch.from_numpy(rng.integers(-20000, 20000, (B, 1, H, D), dtype=np.int32)).to(dev)
                   for _ in range(3))
        extra = dict(
            qkv_inp_scale=torch.from_numpy(((rng.random(B) + 0.5) * 2e-3).astype(np.float32)).to(dev),
            q_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            k_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            v_weight_scale=torch.from_numpy((rng.random(H * D) * 3e-2 + 1e-3).astype(np.float32)).to(dev),
            out_int8=torch.empty(B, H * D, dtype=torch.int8, device=dev),
            out_scale=torch.empty(B, dtype=torch.float32, device=dev))
    ios = [op.make_io(q, k, v, kc, vc, freq, out, start_pos=start_pos, start_pos_per_seq=pos_d,
                      max_start_pos=start_pos if ragged else -1, attn_mask=mask_d, **extra) for kc, vc in caches]
    stream = torch.cuda.current_stream(dev)

    def run(n, passes=3):
        for i in range(n):
            st = op.launch(ios[i % copies], passes=passes, stream=stream)
            if st != 0:
                raise capi.FlAttnError(st, capi.strerror(st))

    # ---- timed regions: W warm-up steps, then `repeats` regions of exactly K steps each between two
    # events on the launch stream; the median region is reported
    run(warmup)
    torch.cuda.synchronize()
    h0 = time.perf_counter()
    step_ms, step_all = time_region(torch, stream, run, steps, repeats)
    host_ms = (time.perf_counter() - h0) * 1e3
    out_gpu = out.cpu().numpy().copy()

    # ---- the streaming kernel alone (pass 1), same launches, same stream.  When the step is one launch
    # (no split, or a split merged inside the kernel) that launch IS the step.
    launches = 1 if plan.two_pass == 0 or (plan.two_pass == 2 and not two_launches) else 2
    one_launch = launches == 1 and segment == "attention"
    if one_launch:
        kern_ms, kern_all = step_ms, step_all
    else:
        run(max(3, warmup // 4), passes=1)
        torch.cuda.synchronize()
        kern_ms, kern_all = time_region(torch, stream, lambda n: run(n, passes=1), steps, repeats)

    # ---- the same step replayed from a HIP graph (how a serving loop hides launch gaps): G steps per
    # graph, rotating over the cache copies like the eager loop; reported beside the eager figure
    graph_us = None
    if graph_steps > 0:
        G = max(copies, graph_steps // copies * copies)
        side = torch.cuda.Stream(device=dev)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                cs = torch.cuda.current_stream(dev)
                for i in range(G):
                    st = op.launch(ios[i % copies], stream=cs)
                    if st != 0:
                        raise capi.FlAttnError(st, capi.strerror(st))
        torch.cuda.synchronize()
        reps = max(1, steps // G)
        for _ in range(2):
            g.replay()
        torch.cuda.synchronize()
        graph_ms, _ = time_region(torch, stream, lambda n: [g.replay() for _ in range(n)], reps, repeats)
        graph_us = graph_ms / G * 1e3
        if not np.array_equal(out.cpu().numpy(), out_gpu):
            raise RuntimeError("HIP-graph replay and eager step disagree")

    alg = algorithmic_bytes(B, H, D, e, sum_ctx, has_mask=mask_h is not None, mean_ctx=sum_ctx / B)
    res = dict(
        name=name, B=B, H=H, D=D, L=L, dtype=w["dtype"], ragged=ragged, mask=mask, copies=copies, sum_ctx=sum_ctx,
        max_ctx=max_ctx, nsplit=plan.nsplit, chunk_rows=plan.chunk_rows,
        launches_per_step=launches + (1 if segment == "int32-int8" else 0),
        alg_bytes=alg, step_ms=step_ms, step_ms_all=step_all, kern_ms=kern_ms, kern_ms_all=kern_all,
        graph_us=graph_us, host_ms=host_ms, gen_s=gen_s, cpu=None)

    # ---- CPU baseline: the scalar oracle on the same inputs.  The full batch when one single-thread pass
    # stays within a few seconds (the headline does: ~1.2 s), else the leading sequences.
    if cpu:
        from oracle import ref  # checker / baseline only
        per_seq = 2 * H * D * e * (sum_ctx / B)
        ns = args.cpu_seqs or max(1, min(B, int(round(2.2e9 / per_seq))))
        sl = slice(0, ns)
        pos_s = pos_h[sl] if ragged else None
        sample_bytes = algorithmic_bytes(ns, H, D, e, int(lens[sl].sum()), has_mask=mask_h is not None,
                                         mean_ctx=float(lens[sl].mean()))

        def cpu_leg(threads, budget_s, min_reps, max_reps):
            kc_s, vc_s = kc_h[sl].copy(), vc_h[sl].copy()
            times, r = [], None
            while len(times) < min_reps or (sum(times) < budget_s and len(times) < max_reps):
                t1 = time.perf_counter()
                r = ref.decode_attn(q_h[sl], k_h[sl], v_h[sl], kc_s, vc_s, freq_h, start_pos=start_pos,
                                    start_pos_per_seq=pos_s, attn_mask=mask_h, threads=threads)
                times.append(time.perf_counter() - t1)
            return r, median(times), len(times), sum(times)

        out_ref, cpu_1t, reps_1t, total_1t = cpu_leg(1, 8.0, 3, 50)
        nthreads = max(1, min(16, os.cpu_count() or 1))
        _, cpu_nt, reps_nt, total_nt = cpu_leg(nthreads, 4.0, 3, 50)
        res["cpu"] = {
            "value": round(sample_bytes / cpu_1t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": (f"all {B} sequences" if ns == B else f"first {ns} of {B} sequences") +
                      f" of the same seeded inputs ({sample_bytes / 1e6:.0f} MB algorithmic per pass), scalar oracle, "
                      f"1 thread, median of {reps_1t} passes ({total_1t:.1f} s of CPU work)",
            "us_per_step": round(cpu_1t * B / ns * 1e6, 1),
            "openmp": {"value": round(sample_bytes / cpu_nt / 1e9, 4), "unit": "GB/s", "cores": nthreads,
                       "passes": reps_nt, "us_per_step": round(cpu_nt * B / ns * 1e6, 1)},
            "gpu_vs_oracle_max_abs_err": float(np.abs(out_gpu[sl] - out_ref).max()),
        }
    del caches, ios, op
    torch.cuda.empty_cache()
    return res


def summary(res):
    """The figures of one workload as they appear under other_configs."""
    gbps = res["alg_bytes"] / (res["step_ms"] * 1e-3) / 1e9
    return {
        "workload": describe(res), "us_per_step": round(res["step_ms"] * 1e3, 2), "GBps": round(gbps, 1),
        "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "nsplit": res["nsplit"],
        "launches_per_step": res["launches_per_step"], "algorithmic_bytes_per_step": res["alg_bytes"],
        "us_per_step_all_regions": [round(x * 1e3, 2) for x in res["step_ms_all"]],
    }


def describe(res):
    return (f"{res['name']}: decode self-attention step, B={res['B']} H={res['H']} D={res['D']} "
            + (f"ragged ctx U[1,{res['L']}] (sum {res['sum_ctx']})" if res["ragged"] else f"ctx={res['max_ctx']}")
            + f" L={res['L']} {res['dtype']} KV cache, RoPE at position, "
            + {"none": "no mask", "causal": "causal additive mask row (0 / -FLT_MAX)",
               "strict": "the reference driver's strict mask row (new token hidden)"}[res["mask"]])


def calibrate(args) -> int:
    """Measurement-only legs: what the memory system, the matrix cores and the launch path of this
    machine sustain (kernels of libfl_calib.so, none of them part of the attention path)."""
    import ctypes as C

    import torch

    from fasterllama_amd import build
    if build.is_stale("calib"):
        build.build_calib()
    lib = C.CDLL(build.outputs("calib"))
    lib.fl_calib_stream_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.fl_calib_mfma.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.fl_calib_empty.argtypes = [C.c_void_p]
    lib.fl_calib_stream_read_two.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p]
    lib.fl_calib_coexec.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.fl_calib_attn_loop.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev)
    sp = C.c_void_p(stream.cuda_stream)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)

    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ms, _ = time_region(torch, stream, lambda k: [fn() for _ in range(k)], n, 5)
        return ms

    def ok(rc):
        if rc != 0:
            raise RuntimeError(f"calibration launch failed: hipError {rc}")

    out = {"calib": args.calib}
    if args.calib == "copy":
        n = 1 << 28  # 2^28 floats = 1 GiB read + 1 GiB written per launch
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        out.update(bytes_read_per_launch=n * 4, bytes_written_per_launch=n * 4, launches=5)
    elif args.calib == "read":
        nbytes = 2 << 30  # the headline step reads 2 GiB of K and V
        buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        buf.random_(0, 256)
        rows = []
        for blocks in (256, 512, 2048, 8192):
            for nt in (0, 1):
                ms = timed(lambda: ok(lib.fl_calib_stream_read(buf.data_ptr(), nbytes, blocks, nt, sink.data_ptr(), sp)), 20)
                rows.append({"workgroups": blocks, "loads": "nt" if nt else "plain", "us": round(ms * 1e3, 1),
                             "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)})
        for blocks in (2048, 8192):  # the decode step's own pattern: K rows and V rows, two streams per workgroup
            ms = timed(lambda: ok(lib.fl_calib_stream_read_two(buf.data_ptr(), nbytes, blocks, sink.data_ptr(), sp)), 20)
            rows.append({"workgroups": blocks, "loads": "nt, two streams of 4 loads per lane (K rows, V rows)", "us": round(ms * 1e3, 1),
                         "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)})
        # the small configurations: what a launch that only READS 64 / 128 / 256 MiB takes, back to back, each launch
        # on a different slice of the buffer (nothing cache resident) — the floor for configurations 4 and 2
        small = []
        for mib in (64, 128, 256):
            n = mib << 20
            slices = nbytes // n
            state = {"i": 0}

            def one(n=n, slices=slices, state=state):
                state["i"] = (state["i"] + 1) % slices
                ok(lib.fl_calib_stream_read(buf.data_ptr() + state["i"] * n, n, 256, 1, sink.data_ptr(), sp))
            ms = timed(one, 200)
            small.append({"MiB": mib, "workgroups": 256, "loads": "nt", "us": round(ms * 1e3, 2), "GBps": round(n / (ms * 1e-3) / 1e9, 1)})
        out.update(bytes=nbytes, pattern="128-bit loads, 8 per lane in flight, one contiguous slice per workgroup", results=rows,
                   small_launches=small)
    elif args.calib == "mfma":
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        rows = []
        for fp32, iters, flop in ((0, 20000, 2 * 32 * 32 * 16), (1, 20000, 2 * 32 * 32 * 2)):
            for wgs_per_cu in (1, 2):
                for rnd in (0, 1):
                    blocks = cus * wgs_per_cu
                    ms = timed(lambda: ok(lib.fl_calib_mfma(fp32, blocks, iters, rnd, sink.data_ptr(), sp)), 5)
                    flops = blocks * 4 * 4 * iters * flop
                    rows.append({"mfma": "v_mfma_f32_32x32x2_f32" if fp32 else "v_mfma_f32_32x32x16_f16",
                                 "waves_per_simd": wgs_per_cu, "operands": "random in [-2,2]" if rnd else "zeros",
                                 "TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1)})
        out.update(compute_units=cus, results=rows)
    elif args.calib == "coexec":
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        iters = 20000
        rows = []
        for n_cu in (cus // 16, cus):
            row = {"compute_units_busy": n_cu}
            for what, name in ((1, "matrix_wave_alone"), (2, "vector_wave_alone"), (3, "both_on_one_simd")):
                ms = timed(lambda: ok(lib.fl_calib_coexec(what, n_cu, iters, sink.data_ptr(), sp)), 3)
                row[name + "_ns_per_block"] = round(ms * 1e6 / iters, 1)
            rows.append(row)
        out.update(block="matrix wave: 8 dependent v_mfma_f32_32x32x16_f16 (256 cycles); vector wave: 48 v_fma_f32 + "
                         "16 v_exp_f32 on 16 independent values; one wave of each kind per SIMD, one workgroup per CU",
                   results=rows)
    elif args.calib == "attnloop":
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        tiles = 1200
        rows = []
        for variant, name, qpw, per_cu in ((0, "32 queries per wave, 2 waves per SIMD (the kernel's shape)", 1, 2),
                                           (1, "the same without the softmax", 1, 2),
                                           (2, "64 queries per wave, 1 wave per SIMD, compiler's order", 2, 1),
                                           (3, "64 queries per wave, one MFMA per six vector instructions (scheduling groups)", 2, 1),
                                           (4, "64 queries per wave without the softmax", 2, 1)):
            ms = timed(lambda: ok(lib.fl_calib_attn_loop(variant, cus, tiles, sink.data_ptr(), sp)), 2)
            wave_tiles = cus * per_cu * 4 * tiles * qpw
            rows.append({"variant": name, "us": round(ms * 1e3, 1),
                         "TFLOPs": round(wave_tiles * 16 * 32768 / (ms * 1e-3) / 1e12, 1),
                         "ns_per_32x32_tile_per_simd": round(ms * 1e6 / (wave_tiles / (4 * cus)), 1)})
        out.update(loop="tile loop of prefill_attn_f16_kernel at D=128 on LDS-resident key tiles: per 32-query x 32-key tile "
                        "16 x v_mfma_f32_32x32x16_f16 (512 matrix cycles), base-2 online softmax, 8 ds_read_b128 + 16 "
                        "ds_read_b64_tr_b16, one workgroup barrier", results=rows)
    elif args.calib == "launch":
        ms = timed(lambda: ok(lib.fl_calib_empty(sp)), 2000)
        out.update(empty_kernel_us_per_launch=round(ms * 1e3, 3),
                   note="back-to-back launches of an empty kernel on one stream, HIP events around 2000 of them")
    print(json.dumps(out), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=5,
                    help="timed regions of --steps steps each; the median region is reported")
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS) + sorted(PREFILL_WORKLOADS) + ["all"],
                    help="'all' prints one JSON line per configuration cfg1..cfg5 (each in a child process)")
    ap.add_argument("--nsplit", type=int, default=0, help="force the context split count (0 = library's choice)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--graph-steps", type=int, default=20,
                    help="also time the step replayed from a HIP graph of this many steps (0 = skip)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the other_configs object (the remaining configurations, measured in the same run "
                         "with the headline workload)")
    ap.add_argument("--calib", choices=["copy", "read", "mfma", "coexec", "attnloop", "launch"],
                    help="measurement-only legs, then exit.  copy: a plain 1 GiB -> 1 GiB elementwise copy (for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings); read: 2 GiB streaming read, plain and non-temporal "
                         "loads; mfma: register-only MFMA loops; coexec: a matrix wave and a vector wave per SIMD, alone and together, "
                         "on a sixteenth of the CUs and on all of them; attnloop: the prompt-phase kernel's tile loop on LDS-resident tiles, "
                         "with and without the softmax, 32 or 64 queries per wave; launch: empty-kernel launch cadence")
    ap.add_argument("--calib-copy", action="store_true", help="same as --calib copy")
    ap.add_argument("--cpu-seqs", type=int, default=0, help="sequences in the CPU sample (0 = auto)")
    ap.add_argument("--prefill-mask", default="causal", choices=["causal", "causal-1e5", "block-causal", "none"],
                    help="prompt-phase workloads: additive causal mask with -FLT_MAX (the reference's driver) or "
                         "-1e5 (its kernel harness) above the diagonal, or no mask")
    ap.add_argument("--prefill-classify-per-call", action="store_true",
                    help="prompt-phase workloads: classify the mask's tiles inside every step instead of once per mask")
    ap.add_argument("--prefill-fast-qk", action="store_true",
                    help="prompt-phase fp16 workloads: FL_ATTN_FLAG_FAST_PROMPT_QK (queries as one fp16 value)")
    ap.add_argument("--mask", default="none", choices=["none", "causal", "strict"],
                    help="decode workloads: additive mask [L, L] with row stride L, row start_pos is used "
                         "(open_decoder.cu:207): causal = 0 up to and including the new token, -FLT_MAX beyond; "
                         "strict = the reference driver's mask, which also hides the new token "
                         "(samples/llama_fp16.cu:73-81)")
    ap.add_argument("--two-launches", action="store_true",
                    help="decode workloads: skip fl_decode_attn_workspace_init, so that a split context is merged "
                         "by a second launch instead of inside the streaming kernel")
    ap.add_argument("--opendecoder-loop", action="store_true",
                    help="time OpenDecoder::forward in the reference driver's layer loop at the workload's shape "
                         "(fasterllama_amd/lib/open_decoder_bench), print its JSON object and exit")
    ap.add_argument("--segment", default="attention", choices=["attention", "int32-int8"],
                    help="attention: q/k/v in the cache dtype -> float output (the headline metric). "
                         "int32-int8: the whole reference segment, int32 GEMM accumulators + scales in, "
                         "per-token INT8 + scale out (implies --no-cpu)")
    args = ap.parse_args()
    if args.calib_copy:
        args.calib = "copy"
    if args.repeats < 1 or args.steps < 1:
        ap.error("--steps and --repeats must be positive")

    if args.workload == "all":
        import subprocess
        rc = 0
        for w in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5"):
            cmd = [sys.executable, os.path.abspath(__file__), "--workload", w, "--steps", str(args.steps),
                   "--warmup", str(args.warmup), "--seed", str(args.seed), "--no-others"] + (["--no-cpu"] if args.no_cpu else [])
            rc |= subprocess.run(cmd).returncode
        return rc

    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no cross-GPU exchange); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    from fasterllama_amd import capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    if args.calib:
        return calibrate(args)
    if args.opendecoder_loop:
        w = WORKLOADS.get(args.workload)
        if w is None or w.get("ragged") or w["dtype"] != "f16":
            print("bench.py: --opendecoder-loop needs a uniform fp16 decode workload", file=sys.stderr)
            return 2
        print(json.dumps(opendecoder_loop(w["B"], w["H"], w["D"], w["L"], w["ctx"] - 1, w["copies"], 20)), flush=True)
        return 0
    if args.workload in PREFILL_WORKLOADS:
        return bench_prefill(args)
    capi.load()  # fails loudly when the HIP library is missing

    if args.segment == "int32-int8":
        args.no_cpu = True
    res = measure_decode(args.workload, args, args.steps, args.warmup, args.repeats, mask=args.mask,
                         graph_steps=args.graph_steps, cpu=not args.no_cpu, two_launches=args.two_launches,
                         segment=args.segment, nsplit=args.nsplit)
    gbps = res["alg_bytes"] / (res["step_ms"] * 1e-3) / 1e9
    kern_gbps = res["alg_bytes"] / (res["kern_ms"] * 1e-3) / 1e9
    traffic, traffic_src = measured_traffic(args.workload, args.mask)

    # ---- the other configurations and the masked headline, measured in the same run (shorter regions)
    others = None
    if args.workload == HEADLINE and not args.no_others and args.mask == "none" and args.segment == "attention":
        others = {}
        o_steps, o_rep = max(10, min(args.steps, 50)), max(3, min(args.repeats, 3))
        for key, name, mask in (("cfg1", "cfg1", "none"), ("cfg2", "cfg2", "none"), ("cfg4", "cfg4", "none"),
                                ("cfg5", "cfg5", "none"), ("cfg3_causal_mask", "cfg3", "causal"),
                                ("cfg3_strict_mask", "cfg3", "strict"),
                                ("cfg3_f32_caches", "x7b_f32", "none")):  # the headline shape in the reference's cache type
            others[key] = summary(measure_decode(name, args, o_steps, max(3, args.warmup // 2), o_rep, mask=mask))
        # the prompt phase of the same block (matrix-core bound: another roofline), reference driver's causal mask
        saved = (args.prefill_mask, args.prefill_fast_qk, args.prefill_classify_per_call)
        args.prefill_mask, args.prefill_fast_qk, args.prefill_classify_per_call = "causal", False, False
        for name in ("prefill_7b_b8_s1024", "prefill_7b_b8_s1024_f32", "prefill_7b_b1_s4096"):
            # (60 warm-up steps: the clock settles only after some 10 ms of matrix load; the first regions of a cold run read 10-15 % slow)
            others[name] = prefill_summary(measure_prefill(args, name, 50, 60, 5))
        args.prefill_mask, args.prefill_fast_qk, args.prefill_classify_per_call = saved
        # OpenDecoder::forward under the reference driver's call pattern, at the small (B=1, ctx 4096) and the headline shape
        others["opendecoder_loop_cfg4"] = opendecoder_loop(1, 32, 128, 4096, 4095, 12, 20)
        others["opendecoder_loop_cfg3"] = opendecoder_loop(64, 32, 128, 2048, 2047, 1, 20)

    line = {
        "metric": "decode-attn us/step + HBM GB/s (% peak), LLaMA2-7B heads b=64 ctx=2048 fp16"
                  if args.workload == HEADLINE else f"decode-attn us/step + HBM GB/s (% peak), {args.workload}",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "repeats": args.repeats,
        "ms_per_step": round(res["step_ms"], 6),
        "us_per_step": round(res["step_ms"] * 1e3, 2),
        "us_per_step_all_regions": [round(x * 1e3, 2) for x in res["step_ms_all"]],
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 storage / f32 accumulate" if res["dtype"] == "f16" else "f32",
        "data": "synthetic (seeded splitmix64 + Box-Muller N(0,1), seed %d)" % args.seed,
        "config": {
            "workload": describe(res),
            "batch": res["B"], "heads": res["H"], "head_dim": res["D"], "ctx": res["max_ctx"] if not res["ragged"] else None,
            "sum_ctx": res["sum_ctx"], "cache_rows": res["L"], "cache_copies_rotated": res["copies"],
            "nsplit": res["nsplit"], "chunk_rows": res["chunk_rows"], "launches_per_step": res["launches_per_step"],
            "algorithmic_bytes_per_step": res["alg_bytes"],
            "segment": args.segment,
            "timing": f"median of {args.repeats} regions of {args.steps} steps after {args.warmup} warm-up steps, HIP events on the launch stream",
        },
        "roofline": {
            "bound": "hbm", "achieved": round(kern_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(kern_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic, "traffic_source": traffic_src,
            "kernel": "decode_attn_split_kernel", "kernel_us": round(res["kern_ms"] * 1e3, 2),
        },
        "cpu_baseline": res["cpu"],
        "other_configs": others,
        "hip_graph_us_per_step": None if res["graph_us"] is None else round(res["graph_us"], 2),
        "host_ms_total": round(res["host_ms"], 3),
        "input_gen_s": round(res["gen_s"], 2),
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
