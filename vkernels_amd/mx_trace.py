"""Where a workgroup of the prefill kernel spends its time: runs one fused layer on a
profiling build of the library (trace points compiled in) and prints the duration of the
kernel's phases over all workgroups of one stage.

    python -m vkernels_amd.build --quiet --define VK_MX_TRACE --out /tmp/vk_trace
    VKERNELS_LIB=/tmp/vk_trace/libvkernels_hip.so python -m vkernels_amd.mx_trace c3:16384 --stage 1

Times are from the device's 100 MHz clock, read by thread 0 of each workgroup."""
from __future__ import annotations

import argparse
import ctypes

import numpy as np


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("workload", help="config:T, e.g. c3:16384")
    ap.add_argument("--stage", type=int, default=1, choices=(0, 1))
    ap.add_argument("--split-terms", type=int, default=0, choices=(0, 2, 3),
                    help="0 = the library's default (3 FP6 terms in the first stage, 2 in the second)")
    ap.add_argument("--w4a4", action="store_true")
    ap.add_argument("--epilogue", default="plain", choices=("plain", "bias_limit", "situ_bias"),
                    help="as bench.py's: both biases and swiglu_limit 7.0, or SiTU (beta 3, linear_beta 20) and both biases")
    args = ap.parse_args()

    import torch
    from vkernels_amd import synth
    from vkernels_amd import vllm_experts as ve

    lib = ve.load_libvkernels_hip()
    if not hasattr(lib, "vk_debug_mx_trace"):
        raise SystemExit("this libvkernels_hip.so has no trace points: build one with --define VK_MX_TRACE "
                         "and point VKERNELS_LIB at it")
    lib.vk_debug_mx_trace.argtypes = [ctypes.c_void_p, ctypes.c_int]
    name, t_str = args.workload.split(":")
    cfg, T = synth.CONFIGS[name], int(t_str)
    dev = torch.device("cuda", 0)
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, 5, device=dev)
    epi = {}
    if args.epilogue != "plain":
        epi.update(b13=torch.from_numpy((synth.rand_normal((cfg.E, 2 * cfg.I), 5, 21) * 0.5).astype(np.float32)).to(dev),
                   b2=torch.from_numpy((synth.rand_normal((cfg.E, cfg.H), 5, 22) * 0.5).astype(np.float32)).to(dev))
        if args.epilogue == "bias_limit":
            epi.update(swiglu_limit=7.0)
        else:
            epi.update(activation="situ", beta=3.0, linear_beta=20.0)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, prepack=True, split_terms=args.split_terms or None,
                         w4a4=args.w4a4, **epi)
    a_bits = synth.make_activations(T, cfg.H, 5)
    A = torch.from_numpy(a_bits.view(np.int16)).view(torch.bfloat16).to(dev)
    logits = torch.from_numpy(synth.make_logits(cfg.logits, T, cfg.E, 5, a_bits, cfg.H)).to(dev)
    ids, tw = fe.route(logits, cfg.top_k, True)
    for _ in range(3):
        fe.apply(A, ids, tw)
    torch.cuda.synchronize()
    n_wg = 1 << 17   # more than any grid of the kernel at the sizes this is used for
    buf = torch.zeros(n_wg * 8, dtype=torch.int64, device=dev)
    lib.vk_debug_mx_trace(buf.data_ptr(), args.stage)
    fe.apply(A, ids, tw)
    torch.cuda.synchronize()
    lib.vk_debug_mx_trace(None, args.stage)

    t = buf.cpu().numpy().reshape(n_wg, 8)
    t = t[(t[:, 0] != 0) & (t[:, 1] != 0)]          # workgroups with routed rows
    t0 = t[:, 0].min()
    entry, listed, kdone, passed, done, first = [(t[:, i] - t0) / 100.0 for i in (0, 1, 2, 3, 4, 5)]
    print(f"{args.workload} stage {args.stage}: {len(t)} workgroups with rows, kernel span {done.max():.0f} us")
    for label, d in (("entry -> rows listed", listed - entry), ("K loop", kdone - listed),
                     ("barrier", passed - kdone), ("epilogue", done - passed),
                     ("  its first row tile", first - passed), ("workgroup", done - entry)):
        print(f"  {label:22s} mean {d.mean():6.2f}  median {np.median(d):6.2f}  p95 {np.percentile(d, 95):6.2f} us")
    cu = ((t[:, 6] >> 8) & 0xFF) | ((t[:, 7] & 0xF) << 8)   # compute unit, shader array and engine; XCC
    gaps = []
    for c in np.unique(cu):
        idx = np.where(cu == c)[0]
        o = idx[np.argsort(entry[idx])]
        gaps.extend((entry[o][1:] - done[o][:-1]).tolist())
    gaps = np.array(gaps)
    print(f"  {len(np.unique(cu))} compute units; gap between consecutive workgroups on one: "
          f"mean {gaps.mean():.2f} median {np.median(gaps):.2f} us")


if __name__ == "__main__":
    main()
