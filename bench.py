#!/usr/bin/env python3
"""Benchmark of the fused MXFP4 MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1:64] [--prefill c3:16384]

A step is one pass of the whole hot path over one batch of synthetic tokens
already resident in HBM: router -> on-device alignment -> gate/up grouped GEMM
+ SwiGLU -> down grouped GEMM + combine, all through the C ABI of
libvkernels_hip.so on one stream.

The metric has two halves, and one JSON line carries both:

* the top-level fields are the decode-shaped workload the metric is quoted on
  (hidden 2880, intermediate 2880, 32 experts, top-4, T = 64), HBM bound.
  `roofline` is its dominant kernel (the gate/up GEMM, two thirds of the
  weight bytes): algorithmic HBM bytes per launch over its mean duration,
  measured with events on the launch stream in a second loop of the same
  steps, against the 8 TB/s peak.  Weight sets are rotated between steps so
  that the 256 MB Infinity Cache cannot serve the 423 MB of weights twice.
  The weights are prepacked at load time and the raw tensors let go of (one
  copy: the decode kernels stream the prepacked form; --no-prepack measures
  the raw form, --keep-raw keeps both);
* `prefill` is the prefill-shaped workload that is bound by the matrix cores
  (hidden 7168, intermediate 2048, 256 experts, top-8, T = 16384) on weights
  prepacked at load time: tokens/s of the whole step and a `roofline` whose
  `achieved` is the layer's algorithmic flops (6 T k H I) over the mean
  event-timed duration of the fused call, against the dense FP4 peak.

`cpu_baseline` times the reference's CPU oracle (or this repository's
restatement when the reference build is absent) on a bounded sample of the
decode workload, single-threaded and on all host cores.
"""
from __future__ import annotations

import argparse
import ctypes
import hashlib
import json
import os
import re
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
FP4_PEAK_TFLOPS = 10100.0
METRIC = "MoE layer tokens/s; % HBM BW roofline (decode), % FP4 MFMA peak (prefill)"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c1:64", help="config:T of the top-level record, e.g. c1:64, c2:512")
    ap.add_argument("--prefill", default="c3:16384",
                    help="config:T of the `prefill` record (prepacked weights); 'none' skips it")
    ap.add_argument("--split-terms", type=int, default=0, choices=(0, 2, 3),
                    help="FP6 terms per activation on the prepacked path: 0 = the library's default "
                         "(3 in the first stage, 2 in the second), 2 or 3 = that many in both")
    ap.add_argument("--no-prepack", action="store_true", help="raw weights only, also for prefill sizes")
    ap.add_argument("--keep-raw", action="store_true",
                    help="keep the raw weight tensors beside the prepacked form (the default lets go of them: "
                         "one copy of the weights, every kernel reads the prepacked form)")
    ap.add_argument("--no-workspace", action="store_true",
                    help="call the reference's own symbol (no workspace, raw weights)")
    ap.add_argument("--no-modes", action="store_true",
                    help="skip the prefill record's other arithmetic modes (2 <-> 3 terms, W4A4)")
    ap.add_argument("--w4a4", action="store_true", help="top-level record in the W4A4 mode (prefill sizes)")
    ap.add_argument("--epilogue", default="plain", choices=("plain", "bias_limit", "situ_bias"),
                    help="what the first stage's epilogue applies besides the activation: nothing; both "
                         "biases and swiglu_limit 7.0; the SiTU activation (beta 3, linear_beta 20) and both biases")
    ap.add_argument("--weight-sets", type=int, default=0, help="0 = enough to exceed 1 GiB")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the HIP-graph replay of the decode step (`graph_ms_per_step`)")
    ap.add_argument("--block-size", type=int, default=0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 512 MiB device copy three times, so that a profiler's "
                         "FETCH_SIZE / WRITE_SIZE counters can be scaled by a kernel of known traffic")
    return ap.parse_args()


def sources_digest() -> str:
    """Digest of the kernel sources, comments and white space left out: names the code a
    profile was taken on."""
    h = hashlib.sha256()
    for path in sorted((ROOT / "vkernels_amd" / "csrc").iterdir()):
        text = path.read_text(errors="replace")
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        h.update(path.name.encode())
        h.update("".join(text.split()).encode())
    return h.hexdigest()[:16]


def measured_traffic(workload: str):
    """HBM bytes per launch of the workload's dominant kernel from the profiler's
    FETCH_SIZE / WRITE_SIZE counters (profiles/traffic.json, written when the build
    was profiled); None when the kernel sources have changed since."""
    path = ROOT / "profiles" / "traffic.json"
    if not path.is_file():
        return None
    try:
        rec = json.loads(path.read_text()).get(workload)
    except (OSError, ValueError):
        return None
    if not rec or rec.get("sources_sha16") != sources_digest():
        return None
    return rec.get("traffic_bytes")


def cpu_baseline(cfg, T, seed, budget_s=12.0):
    """Reference CPU oracle on a bounded sample of the workload: one thread (the
    reference oracle is single-threaded) and all host cores (OpenMP over tiles,
    bit-identical for any thread count)."""
    import numpy as np
    import oracle
    from vkernels_amd import synth

    use_ref = oracle.have_ref()
    t_cpu = min(T, 64)
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed).numpy()
    A = synth.make_activations(t_cpu, cfg.H, seed)
    lg = synth.make_logits(cfg.logits, t_cpu, cfg.E, seed, A, cfg.H)

    def timed(threads, ref):
        oracle.set_threads(threads)
        times = []
        t_begin = time.perf_counter()
        while len(times) < 3 and (not times or time.perf_counter() - t_begin < budget_s):
            t0 = time.perf_counter()
            oracle.moe_layer(A, lg, *w, cfg.top_k, use_ref=ref)
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2], len(times)

    one, n_one = timed(1, use_ref)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores) or cores))
    many, n_many = timed(cores, False)  # the OpenMP build is this repository's restatement
    oracle.set_threads(1)
    return {
        "value": t_cpu / one, "unit": "tokens/s", "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": f"{cfg.name} T={t_cpu}: router + align + fused layer, median of "
                  f"{n_one} runs, {one * 1e3:.1f} ms each",
        "all_cores": {"value": t_cpu / many, "unit": "tokens/s", "cores": cores, "kind": "port",
                      "sample": f"same sample, {many * 1e3:.1f} ms (median of {n_many})"},
        "host_cpus": os.cpu_count(),
    }


def run_workload(args, workload, steps, warmup, prepack, split_terms=None, w4a4=False):
    """Times one workload; returns the record's fields.  split_terms / w4a4 choose the
    arithmetic of the prepacked path (default: args.split_terms FP6 terms per bf16
    activation; w4a4: activations quantised to MXFP4 as the reference's mxfp4_moe_quant
    does, one FP4 x FP4 MFMA per product)."""
    import numpy as np
    import torch
    from vkernels_amd import synth
    from vkernels_amd import vllm_experts as ve

    name, t_str = workload.split(":")
    cfg = synth.CONFIGS[name]
    T = int(t_str)
    seed = synth.config_seed(cfg, T)
    dev = torch.device("cuda", 0)
    H, I, k = cfg.H, cfg.I, cfg.top_k
    prepack = prepack and not args.no_workspace   # at every size: the decode kernels read the prepacked form too
    packed_only = prepack and not args.keep_raw
    terms = args.split_terms if split_terms is None else split_terms   # 0 = the library's default

    per_set = synth.algorithmic_bytes(H, I, cfg.E, k, 0, cfg.E)
    n_sets = args.weight_sets or max(2, -(-(1 << 30) // per_set))
    n_sets = min(n_sets, 8)
    if per_set > (1 << 30):
        n_sets = 1  # one set is already several times the Infinity Cache
    experts = []
    epi = {}
    if args.epilogue != "plain":
        epi.update(b13=torch.from_numpy((synth.rand_normal((cfg.E, 2 * I), seed, 21) * 0.5).astype(np.float32)).to(dev),
                   b2=torch.from_numpy((synth.rand_normal((cfg.E, H), seed, 22) * 0.5).astype(np.float32)).to(dev))
        if args.epilogue == "bias_limit":
            epi.update(swiglu_limit=7.0)
        else:
            epi.update(activation="situ", beta=3.0, linear_beta=20.0)
    for s in range(n_sets):
        w = synth.make_weights(cfg.E, H, I, seed + 7919 * s, device=dev)
        experts.append(ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, prepack=prepack,
                                       split_terms=terms or None, w4a4=w4a4 and prepack,
                                       keep_raw=not packed_only, **epi))
        if packed_only:
            del w
        if args.no_workspace:
            experts[-1].use_workspace = False
    A_bits = synth.make_activations(T, H, seed)
    logits_np = synth.make_logits(cfg.logits, T, cfg.E, seed, A_bits, H)
    A = torch.from_numpy(A_bits.view(np.int16)).view(torch.bfloat16).to(dev)
    logits = torch.from_numpy(logits_np).to(dev)
    out = torch.empty((T, H), dtype=torch.float32, device=dev)
    bs = args.block_size or experts[0].block_size_for(T, k)
    lib = ve.load_libvkernels_hip()
    # the library's own split between its decode and tile kernels
    prefill = bs > 32 or T * k > int(lib.vk_hip_moe_decode_max_rows(cfg.E if prepack else 0, bs))
    lib.vk_hip_moe_gateup_mxfp4_ex.restype = None
    lib.vk_hip_moe_down_mxfp4_ex.restype = None

    def step(i, events=None):
        fe = experts[i % n_sets]
        if events is None:
            if not args.no_workspace:
                # router, alignment and the layer through the library's one call
                fe.route_layer(A, logits, k, block_size=bs, out_fp32=out)
                return
            # router and alignment through the library's one call (one launch at decode sizes)
            ids, w, sids, eids, _, max_em, _ = fe.route_align(logits, k, True, bs)
            fe.apply(A, ids, w, block_size=bs, out_fp32=out, aligned=(sids, eids, max_em))
            return
        ids, w = fe.route(logits, k, True)
        # same launches, with events around the two GEMM stages (decode) or around
        # the fused call (prefill-sized batches, which run with a workspace)
        sids, eids, _, max_em = fe.align(ids, bs)
        if prefill:
            events[0].record()
            events[1].record()
            if args.no_workspace:
                out.zero_()
            fe.fused_call(A, ids, w, sids, eids, max_em, bs, out, overwrite=not args.no_workspace)
            events[2].record()
            return
        out.zero_()
        act = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16, device=dev)
        st = ve._P(torch.cuda.current_stream().cuda_stream)
        e0, e1, e2 = events
        e0.record()
        lib.vk_hip_moe_gateup_mxfp4_ex(
            ve._ptr(A), ve._ptr(fe.w13), ve._ptr(fe.w13_scale), ve._ptr(act), T, H, I,
            k, ve._ptr(sids), ve._ptr(eids), max_em, ve._F(float(fe.swiglu_limit)), fe.activation,
            ve._F(float(fe.beta)), ve._F(float(fe.linear_beta)), ve._ptr(fe.b13), bs,
            ve._ptr(fe.w13_packed), fe.E, st)
        e1.record()
        lib.vk_hip_moe_down_mxfp4_ex(
            ve._ptr(act), ve._ptr(fe.w2), ve._ptr(fe.w2_scale), ve._ptr(w), ve._ptr(out), T,
            H, I, k, ve._ptr(sids), ve._ptr(eids), max_em, ve._ptr(fe.b2), bs, None, ctypes.c_size_t(0),
            ctypes.c_uint(0), ve._ptr(fe.w2_packed), fe.E, st)
        e2.record()

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3

    # The same steps as captured HIP graphs, one per weight set, replayed in rotation: how a
    # serving loop runs decode (the reference's caller captures the layer,
    # src/python/vkernels/vllm_experts.py:142-246).  Decode-sized batches only: beyond, a
    # step is milliseconds and its launches do not matter.
    graph_ms_per_step = None
    if not prefill and not args.no_graph:
        graphs = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for s in range(n_sets):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    step(s)
                graphs.append(g)
        torch.cuda.current_stream().wait_stream(side)
        for i in range(min(warmup, 5)):
            graphs[i % n_sets].replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            graphs[i % n_sets].replay()
        torch.cuda.synchronize()
        graph_ms_per_step = (time.perf_counter() - t0) / steps * 1e3
        del graphs

    # Second loop: the same steps with events around each GEMM stage.
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for i in range(min(warmup, 5)):
        step(i, ev[0])
    torch.cuda.synchronize()
    for i in range(steps):
        step(i, ev[i])
    torch.cuda.synchronize()
    gate_ms = sorted(e[0].elapsed_time(e[1]) for e in ev)
    down_ms = sorted(e[1].elapsed_time(e[2]) for e in ev)
    gate_avg = sum(gate_ms) / len(gate_ms)
    down_avg = sum(down_ms) / len(down_ms)

    ids, _ = experts[0].route(logits, k, True)
    active = int(torch.unique(ids).numel())  # from the actual routing
    gate_bytes = active * (I * H + I * H // 16) + 2 * T * H + 2 * T * k * I
    down_bytes = active * (H * I // 2 + H * I // 32) + 2 * T * k * I + 4 * T * H
    layer_bytes = synth.algorithmic_bytes(H, I, cfg.E, k, T, active)
    flops = synth.algorithmic_flops(H, I, k, T)
    if prefill:
        fused_tflops = flops / (down_avg * 1e-3) / 1e12
        if prepack and w4a4:
            kernel = ("vk_hip_fused_moe_mxfp4_prepacked, W4A4 (quant_rows_w4_kernel x2 + tile_mx_kernel<0,1> + "
                      "tile_mx_kernel<1,1> + combine_kernel)")
            issued = 1.0
        elif prepack:
            t0, t1 = (terms, terms) if terms else (3, 2)
            kernel = (f"vk_hip_fused_moe_mxfp4_prepacked (split_rows_fp6_kernel<{t0}> + tile_mx_kernel<0,{t0}> + "
                      f"split_rows_fp6_kernel<{t1}> + tile_mx_kernel<1,{t1}> + combine_kernel)")
            issued = (2.0 * t0 + t1) / 3.0  # FP4-rate MFMAs per algorithmic product (2/3 of them in stage 0)
        elif args.no_workspace:
            kernel = "vk_hip_fused_moe_mxfp4 (clear of out + tile_gemm_kernel<0> + tile_gemm_kernel<1>, atomics)"
            issued = 4.0
        else:
            kernel = ("vk_hip_fused_moe_mxfp4_ex (split_rows_kernel + tile_wide_kernel<0> + "
                      "tile_wide_kernel<1> + combine_kernel)")
            issued = 4.0  # two FP8-rate MFMAs per product = four at the FP4 rate
        roofline = {
            "bound": "mfma", "kernel": kernel,
            "achieved": fused_tflops, "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": fused_tflops / FP4_PEAK_TFLOPS,
            "traffic": measured_traffic(workload) if prepack and not w4a4 and not terms else None,
            "matrix_rate_frac": issued * fused_tflops / FP4_PEAK_TFLOPS,
            "flops_per_launch": flops, "avg_launch_us": down_avg * 1e3,
            "median_launch_us": down_ms[len(down_ms) // 2] * 1e3,
        }
    else:
        achieved = gate_bytes / (gate_avg * 1e-3) / 1e9
        roofline = {
            "bound": "hbm", "kernel": "stream_resident_kernel<0, ...> (gate/up grouped GEMM + SwiGLU"
                                      + (", weights read from the prepacked form)" if prepack else ")"),
            "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(workload),
            "bytes_per_launch": gate_bytes, "avg_launch_us": gate_avg * 1e3,
            "median_launch_us": gate_ms[len(gate_ms) // 2] * 1e3,
        }
    rec = {
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "graph_ms_per_step": graph_ms_per_step,
        "config": {
            "workload": f"{cfg.name} T={T}: hidden {H}, intermediate {I}, {cfg.E} experts, "
                        f"top-{k}, MXFP4 weights, bf16 activations, {cfg.logits} routing",
            "block_size": bs, "active_experts": active, "weight_sets": n_sets,
            "weights": "prepacked at load time, one copy (the raw tensors let go of)" if packed_only
                       else "prepacked at load time (+ raw)" if prepack else "raw",
            "epilogue": args.epilogue,
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
    if prepack and not prefill:
        rec["config"]["activations"] = "bf16 split exactly into two E4M3 terms per block of 32 (decode kernels)"
    elif prepack:
        rec["config"]["activations"] = (
            "MXFP4 (reference mxfp4_moe_quant), one FP4 x FP4 MFMA per product" if w4a4 else
            f"bf16 as {terms} FP6 E2M3 terms per block of 32 in both stages" if terms else
            "bf16 as FP6 E2M3 terms per block of 32: 3 in the first stage, 2 in the second")
        rec["config"]["split_terms"] = [1, 1] if w4a4 else [terms, terms] if terms else [3, 2]
    del experts
    torch.cuda.empty_cache()
    return rec, cfg, T, seed


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(no collectives are part of the fused MoE path)", file=sys.stderr)
        sys.exit(2)

    import torch
    torch.cuda.set_device(torch.device("cuda", 0))

    rec, cfg, T, seed = run_workload(args, args.workload, args.steps, args.warmup, not args.no_prepack,
                                     w4a4=args.w4a4)
    line = {
        "metric": METRIC,
        "value": rec["value"],
        "unit": rec["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": rec["ms_per_step"],
        "graph_ms_per_step": rec["graph_ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": rec["config"],
        "roofline": rec["roofline"],
        "layer": rec["layer"],
    }
    if args.prefill != "none" and args.prefill != args.workload:
        # fewer steps: a prefill step is milliseconds, and the default run must stay short
        p_steps = max(5, min(args.steps, 20))
        p_rec, _, _, _ = run_workload(args, args.prefill, p_steps, min(args.warmup, 3),
                                      not args.no_prepack)
        if not args.no_prepack and not args.no_modes:
            # the same workload in the path's other two arithmetic modes (see `activations`)
            p_rec["other_modes"] = {}
            others = [("fp6_terms_%d" % t, dict(split_terms=t)) for t in (3, 2) if t != args.split_terms]
            if args.split_terms:
                others.insert(0, ("fp6_terms_3_2", dict(split_terms=0)))
            for key, kw in others + [("w4a4", dict(w4a4=True))]:
                m_rec, _, _, _ = run_workload(args, args.prefill, p_steps, min(args.warmup, 3), True, **kw)
                p_rec["other_modes"][key] = {
                    "value": m_rec["value"], "ms_per_step": m_rec["ms_per_step"],
                    "activations": m_rec["config"]["activations"],
                    "fused_call_us": m_rec["roofline"]["avg_launch_us"],
                    "frac": m_rec["roofline"]["frac"],
                    "matrix_rate_frac": m_rec["roofline"]["matrix_rate_frac"],
                }
        line["prefill"] = p_rec
    if args.copy_calibration:
        dev = torch.device("cuda", 0)
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
