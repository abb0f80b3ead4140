"""Sweep of the decode launch shapes: times every candidate shape of both GEMM stages on
synthetic layers and prints the table the compiled-in rules are set from; with --store
the winners go to the tuning store the library reads (moe_fused.gfx950.tune).

    python -m vkernels_amd.tune_moe                      # the default shapes, markdown to stdout
    python -m vkernels_amd.tune_moe --store ~/.cache/vkernels/tuning --shapes 2880x2880x32x4
    python -m vkernels_amd.tune_moe --packed             # the decode kernels that read the prepacked form

A shape is HIDDENxINTERMEDIATExEXPERTSxTOP_K; each is swept at the token counts of
--tokens.  One stage call is timed with HIP events over `--iters` launches that rotate
weight sets larger than the Infinity Cache; the figure is the median.
Needs a GPU.  Same role as the reference's sweep benches that write the native tuning
store (src/c/vkernels/core/tuning.hpp:1-9).
"""
from __future__ import annotations

import argparse
import statistics
import sys
from pathlib import Path

DEFAULT_SHAPES = ("2880x2880x32x4", "2880x2880x128x4", "4096x1536x64x6", "7168x2048x256x8", "256x512x8x2")
DEFAULT_TOKENS = (1, 8, 32, 64, 128)


def time_stage(torch, ve, lib, fe_sets, stage, A, ids, tw, out, bs, iters):
    dev = A.device
    T, H = A.shape
    k = ids.shape[1]
    fe = fe_sets[0]
    sids, eids, _, max_em = fe.align(ids, bs)
    act = torch.zeros((max_em, fe.ispp), dtype=torch.bfloat16, device=dev)
    st = ve._P(torch.cuda.current_stream().cuda_stream)
    lib.vk_hip_moe_gateup_mxfp4.restype = None
    lib.vk_hip_moe_down_mxfp4.restype = None
    lib.vk_hip_moe_gateup_mxfp4_ex.restype = None
    lib.vk_hip_moe_down_mxfp4_ex.restype = None

    def call(f):
        if f.w13_packed is not None:   # the prepacked form alone
            if stage == 0:
                lib.vk_hip_moe_gateup_mxfp4_ex(ve._ptr(A), None, None, ve._ptr(act), T, H, f.ispp, k, ve._ptr(sids),
                                               ve._ptr(eids), max_em, ve._F(0.0), 0, ve._F(4.0), ve._F(25.0), None,
                                               bs, ve._ptr(f.w13_packed), f.E, st)
            else:
                lib.vk_hip_moe_down_mxfp4_ex(ve._ptr(act), None, None, ve._ptr(tw), ve._ptr(out), T, H, f.ispp, k,
                                             ve._ptr(sids), ve._ptr(eids), max_em, None, bs, None,
                                             ve.ctypes.c_size_t(0), ve.ctypes.c_uint(0), ve._ptr(f.w2_packed),
                                             f.E, st)
            return
        if stage == 0:
            lib.vk_hip_moe_gateup_mxfp4(ve._ptr(A), ve._ptr(f.w13), ve._ptr(f.w13_scale), ve._ptr(act), T, H,
                                        f.ispp, k, ve._ptr(sids), ve._ptr(eids), max_em, ve._F(0.0), 0,
                                        ve._F(4.0), ve._F(25.0), None, bs, st)
        else:
            lib.vk_hip_moe_down_mxfp4(ve._ptr(act), ve._ptr(f.w2), ve._ptr(f.w2_scale), ve._ptr(tw), ve._ptr(out),
                                      T, H, f.ispp, k, ve._ptr(sids), ve._ptr(eids), max_em, None, bs, st)

    for i in range(3):
        call(fe_sets[i % len(fe_sets)])
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for i, (a, b) in enumerate(ev):
        a.record()
        call(fe_sets[i % len(fe_sets)])
        b.record()
    torch.cuda.synchronize()
    return statistics.median(a.elapsed_time(b) for a, b in ev) * 1e3


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", nargs="*", default=list(DEFAULT_SHAPES))
    ap.add_argument("--tokens", nargs="*", type=int, default=list(DEFAULT_TOKENS))
    ap.add_argument("--iters", type=int, default=40)
    ap.add_argument("--store", default=None, help="directory to write moe_fused.gfx950.tune into")
    ap.add_argument("--packed", action="store_true",
                    help="sweep the decode kernels that read the prepacked form (the weights are prepacked "
                         "and the raw tensors let go of); shapes they do not take are skipped")
    ap.add_argument("--block-size", type=int, default=0,
                    help="alignment block of the calls (default: the library's policy, and only batches of "
                         "up to 512 routed rows); 32 with --packed: the chunked decode kernel's two-tile passes")
    args = ap.parse_args()

    import numpy as np
    import torch
    sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
    from vkernels_amd import synth
    from vkernels_amd import vllm_experts as ve

    lib = ve.load_libvkernels_hip()
    ve.moe_tuning_load("/nonexistent")   # compiled-in rules only, whatever the machine's store holds
    dev = torch.device("cuda", 0)
    print("| shape (H x I x E x k) | T | stage | " + "compiled-in rule | best | " + "us per candidate (variant,waves,tiles,depth) |")
    print("|---|---:|---:|---|---|---|")
    for shape in args.shapes:
        H, I, E, k = (int(x) for x in shape.split("x"))
        per_set = E * (H * I * 3 // 2) * 17 // 16
        n_sets = 1 if per_set > (1 << 30) else max(2, -(-(1 << 30) // per_set))
        fe_sets = []
        for s in range(min(n_sets, 8)):
            w = synth.make_weights(E, H, I, 900 + s, device=dev)
            fe_sets.append(ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, prepack=args.packed,
                                           keep_raw=not args.packed))
            del w
        for T in args.tokens:
            if T * k > 512 and not args.block_size:
                continue   # the tile kernels' side of the split: nothing to choose between
            A = torch.from_numpy(synth.make_activations(T, H, 7).view(np.int16)).view(torch.bfloat16).to(dev)
            logits = torch.from_numpy(synth.make_logits("uniform", T, E, 7)).to(dev)
            ids, tw = fe_sets[0].route(logits, k, True)
            out = torch.zeros((T, H), dtype=torch.float32, device=dev)
            bs = args.block_size or ve.default_block_size(T, k)
            for stage, K, ncols in ((0, H, I), (1, I, H)):
                rule, _ = ve.moe_tile_query(stage, K, ncols, min(T * k, 512) if args.block_size else T * k,
                                            packed=args.packed, block_size=bs)
                times = {}
                for cand in ve.moe_tile_candidates(stage):
                    if args.packed and cand[0] == 0:
                        continue   # the tile kernels read the raw tensors
                    ve.moe_tile_set(stage, K, ncols, T * k, cand)
                    lib.vk_set_last_error(0, b"")
                    t = time_stage(torch, ve, lib, fe_sets, stage, A, ids, tw, out, bs, args.iters)
                    if int(lib.vk_last_error_code()) == 0:   # (refused: a shape the packed kernels do not take)
                        times[cand] = t
                if rule not in times:
                    ve.moe_tile_set(stage, K, ncols, T * k, None)
                    continue
                best = min(times, key=times.get)
                # keep the rule's shape unless another is faster by more than the noise of the measurement
                keep = rule if times[rule] <= 1.02 * times[best] else best
                ve.moe_tile_set(stage, K, ncols, T * k, keep if args.store else None)
                cells = " ".join(f"{c}={t:.1f}" for c, t in times.items())
                print(f"| {shape} | {T} | {stage} | {rule} {times[rule]:.1f} | {best} {times[best]:.1f} | {cells} |",
                      flush=True)
        del fe_sets
        torch.cuda.empty_cache()
    if args.store:
        root = Path(args.store).expanduser()
        root.mkdir(parents=True, exist_ok=True)
        (root / "moe_fused.gfx950.tune").write_text(
            ve.moe_tuning_dump().replace("written_by=vk_hip_moe_tuning_dump", "written_by=vkernels_amd.tune_moe"))
        print(f"wrote {root / 'moe_fused.gfx950.tune'}", file=sys.stderr)


if __name__ == "__main__":
    main()
