#!/usr/bin/env python3
"""Benchmark of the fused MXFP4 MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1:64]

A step is one pass of the whole hot path over one batch of synthetic tokens
already resident in HBM: router -> on-device alignment -> clearing `out` ->
gate/up grouped GEMM + SwiGLU -> down grouped GEMM + combine, all through the
C ABI of libvkernels_hip.so on one stream.  The default workload is the
decode-shaped layer the headline metric is quoted on (hidden 2880,
intermediate 2880, 32 experts, top-4, T = 64).  Weight sets are rotated
between steps so that the 256 MB Infinity Cache cannot serve the 423 MB of
expert weights twice.

One JSON line is printed.  `value` is tokens/s of the whole step.  `roofline`
is for the dominant kernel (the gate/up GEMM, two thirds of the weight bytes):
its algorithmic HBM bytes per launch divided by its mean duration, measured
with events on the launch stream in a second loop of the same steps, against
the 8 TB/s peak.  `cpu_baseline` times the reference's CPU oracle (or this
repository's restatement when the reference build is absent) on the same
workload on the host's cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
FP4_PEAK_TFLOPS = 10100.0

# HBM bytes per launch of the gate/up kernel from rocprofv3 FETCH_SIZE and
# WRITE_SIZE counters (two runs of this script under --pmc, scaled by what the
# same counters read for the 512 MiB copy of --copy-calibration: x2.0 and x1.0).
# Counters cannot be read from inside this process, so the figure of the last
# profiled build is recorded here per workload; null for the others.
MEASURED_TRAFFIC = {"c1:64": 309.1e6}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c1:64", help="config:T, e.g. c1:64, c2:512")
    ap.add_argument("--weight-sets", type=int, default=0, help="0 = enough to exceed 1 GiB")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--block-size", type=int, default=0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 512 MiB device copy three times, so that a profiler's "
                         "FETCH_SIZE / WRITE_SIZE counters can be scaled by a kernel of known traffic")
    return ap.parse_args()


def cpu_baseline(cfg, T, seed, steps_budget_s=30.0):
    """Reference CPU oracle on the same workload, single thread."""
    import numpy as np
    import oracle
    from vkernels_amd import synth

    use_ref = oracle.have_ref()
    oracle.set_threads(1)
    # bounded sample: enough tokens for about 10-30 s of single-core work
    t_cpu = min(T, 64)
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed).numpy()
    A = synth.make_activations(t_cpu, cfg.H, seed)
    lg = synth.make_logits(cfg.logits, t_cpu, cfg.E, seed, A, cfg.H)
    times = []
    t_begin = time.perf_counter()
    while len(times) < 3 and (not times or time.perf_counter() - t_begin < steps_budget_s):
        t0 = time.perf_counter()
        oracle.moe_layer(A, lg, *w, cfg.top_k, use_ref=use_ref)
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2]
    return {
        "value": t_cpu / best, "unit": "tokens/s", "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": f"{cfg.name} T={t_cpu}: router + align + fused layer, median of "
                  f"{len(times)} runs, {best * 1e3:.1f} ms each",
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(no collectives are part of the fused MoE path)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from vkernels_amd import synth
    from vkernels_amd import vllm_experts as ve

    name, t_str = args.workload.split(":")
    cfg = synth.CONFIGS[name]
    T = int(t_str)
    seed = synth.config_seed(cfg, T)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    per_set = synth.algorithmic_bytes(cfg.H, cfg.I, cfg.E, cfg.top_k, 0, cfg.E)
    n_sets = args.weight_sets or max(2, -(-(1 << 30) // per_set))
    n_sets = min(n_sets, 8)
    experts = []
    for s in range(n_sets):
        w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed + 7919 * s, device=dev)
        experts.append(ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale))
    A_bits = synth.make_activations(T, cfg.H, seed)
    logits_np = synth.make_logits(cfg.logits, T, cfg.E, seed, A_bits, cfg.H)
    A = torch.from_numpy(A_bits.view(np.int16)).view(torch.bfloat16).to(dev)
    logits = torch.from_numpy(logits_np).to(dev)
    out = torch.empty((T, cfg.H), dtype=torch.float32, device=dev)
    bs = args.block_size or ve.default_block_size(T, cfg.top_k)
    prefill = T * cfg.top_k > 512  # the library's own split between its decode and tile kernels

    def step(i, events=None):
        fe = experts[i % n_sets]
        ids, w = fe.route(logits, cfg.top_k, True)
        if events is None:
            fe.apply(A, ids, w, block_size=bs, out_fp32=out)
            return
        # same launches, with events around the two GEMM stages (decode) or around
        # the fused call (prefill-sized batches, which run with a workspace)
        sids, eids, _, max_em = fe.align(ids, bs)
        if prefill:
            events[0].record()
            events[1].record()
            fe.fused_call(A, ids, w, sids, eids, max_em, bs, out, overwrite=True)
            events[2].record()
            return
        out.zero_()
        act = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16, device=dev)
        st = ve._P(torch.cuda.current_stream().cuda_stream)
        e0, e1, e2 = events
        e0.record()
        lib.vk_hip_moe_gateup_mxfp4(
            ve._ptr(A), ve._ptr(fe.w13), ve._ptr(fe.w13_scale), ve._ptr(act), T, cfg.H, cfg.I,
            cfg.top_k, ve._ptr(sids), ve._ptr(eids), max_em, ve._F(0.0), 0, ve._F(4.0),
            ve._F(25.0), None, bs, st)
        e1.record()
        lib.vk_hip_moe_down_mxfp4(
            ve._ptr(act), ve._ptr(fe.w2), ve._ptr(fe.w2_scale), ve._ptr(w), ve._ptr(out), T,
            cfg.H, cfg.I, cfg.top_k, ve._ptr(sids), ve._ptr(eids), max_em, None, bs, st)
        e2.record()

    lib = ve.load_libvkernels_hip()
    lib.vk_hip_moe_gateup_mxfp4.restype = None
    lib.vk_hip_moe_down_mxfp4.restype = None

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # Second loop: the same steps with events around each GEMM stage.
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for i in range(min(args.warmup, 5)):
        step(i, ev[0])
    torch.cuda.synchronize()
    for i in range(args.steps):
        step(i, ev[i])
    torch.cuda.synchronize()
    gate_ms = sorted(e[0].elapsed_time(e[1]) for e in ev)
    down_ms = sorted(e[1].elapsed_time(e[2]) for e in ev)
    gate_avg = sum(gate_ms) / len(gate_ms)
    down_avg = sum(down_ms) / len(down_ms)

    # active experts from the actual routing
    ids, _ = experts[0].route(logits, cfg.top_k, True)
    active = int(torch.unique(ids).numel())
    H, I, k = cfg.H, cfg.I, cfg.top_k
    gate_bytes = active * (I * H + I * H // 16) + 2 * T * H + 2 * T * k * I
    down_bytes = active * (H * I // 2 + H * I // 32) + 2 * T * k * I + 4 * T * H
    layer_bytes = synth.algorithmic_bytes(H, I, cfg.E, k, T, active)
    flops = synth.algorithmic_flops(H, I, k, T)
    if prefill:
        # events[1]..[2] bracket the whole fused call (split pass + both grouped GEMMs)
        fused_tflops = flops / (down_avg * 1e-3) / 1e12
        roofline = {
            "bound": "mfma", "kernel": "vk_hip_fused_moe_mxfp4_ex (split_rows_kernel + tile_wide_kernel<0> "
                                       "+ tile_wide_kernel<1> + combine_kernel)",
            "achieved": fused_tflops, "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": fused_tflops / FP4_PEAK_TFLOPS, "traffic": None,
            "flops_per_launch": flops, "avg_launch_us": down_avg * 1e3,
            "median_launch_us": down_ms[len(down_ms) // 2] * 1e3,
        }
    else:
        achieved = gate_bytes / (gate_avg * 1e-3) / 1e9
        roofline = {
            "bound": "hbm", "kernel": "stream_resident_kernel<0, ...> (gate/up grouped GEMM + SwiGLU)",
            "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get(args.workload),
            "bytes_per_launch": gate_bytes, "avg_launch_us": gate_avg * 1e3,
            "median_launch_us": gate_ms[len(gate_ms) // 2] * 1e3,
        }

    line = {
        "metric": "MoE layer tokens/s; % HBM BW roofline (decode), % FP4 MFMA peak (prefill)",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{cfg.name} T={T}: hidden {H}, intermediate {I}, {cfg.E} experts, "
                        f"top-{k}, MXFP4 weights, bf16 activations, {cfg.logits} routing",
            "block_size": bs, "active_experts": active, "weight_sets": n_sets,
        },
        "roofline": roofline,
        "layer": {
            "algorithmic_bytes": layer_bytes, "algorithmic_flops": flops,
            "hbm_frac_whole_step": layer_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "fp4_mfma_frac_whole_step": flops / (ms_per_step * 1e-3) / 1e12 / FP4_PEAK_TFLOPS,
            "down_kernel_avg_us": None if prefill else down_avg * 1e3,
            "down_kernel_gbs": None if prefill else down_bytes / (down_avg * 1e-3) / 1e9,
        },
    }
    if args.copy_calibration:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg, T, seed)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
