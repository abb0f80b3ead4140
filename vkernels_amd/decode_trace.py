"""Where a workgroup of the decode kernel spends its time before its weight stream runs:
one decode step on a profiling build of the library (trace points compiled in), then the
duration of the steps of the kernel's start, mean over the workgroups.

    python -m vkernels_amd.build --quiet --define VK_DECODE_TRACE --out /tmp/vk_dtrace
    VKERNELS_LIB=/tmp/vk_dtrace/libvkernels_hip.so python -m vkernels_amd.decode_trace c1:64

Times are from the device's 100 MHz clock, read by thread 0 of each workgroup (wavefront 0)
in the first 16-row pass the workgroup makes."""
from __future__ import annotations

import argparse
import ctypes

import numpy as np

STAGES, WORKGROUPS, SLOTS = 2, 1024, 12
# (label, from slot, to slot)
PHASES = (
    ("entry -> runs listed (wavefront 0)", 0, 5),
    ("-> slice known, barrier", 5, 1),
    ("-> set-up of the loops done", 1, 6),
    ("-> rows and first weight steps asked for", 6, 7),
    ("-> barrier with the previous pass", 7, 8),
    ("-> first rows in, split and written", 8, 9),
    ("-> scales parked", 9, 10),
    ("-> barrier: the stream starts", 10, 3),
    ("stream", 3, 4),
    ("entry -> end", 0, 4),
)


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("workload", nargs="?", default="c1:64", help="config:T of a decode-sized call, e.g. c1:64")
    args = ap.parse_args()

    import torch
    from vkernels_amd import synth
    from vkernels_amd import vllm_experts as ve

    lib = ve.load_libvkernels_hip()
    if not hasattr(lib, "vk_debug_decode_trace"):
        raise SystemExit("this libvkernels_hip.so has no trace points: build one with --define VK_DECODE_TRACE "
                         "and point VKERNELS_LIB at it")
    lib.vk_debug_decode_trace.argtypes = [ctypes.c_void_p]
    lib.vk_debug_decode_trace.restype = ctypes.c_int
    name, t_str = args.workload.split(":")
    cfg, T = synth.CONFIGS[name], int(t_str)
    dev = torch.device("cuda", 0)
    sets = [synth.make_weights(cfg.E, cfg.H, cfg.I, 5 + i, device=dev) for i in range(3)]  # > the Infinity Cache
    fes = [ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale) for w in sets]
    a_bits = synth.make_activations(T, cfg.H, 5)
    A = torch.from_numpy(a_bits.view(np.int16)).view(torch.bfloat16).to(dev)
    logits = torch.from_numpy(synth.make_logits(cfg.logits, T, cfg.E, 5, a_bits, cfg.H)).to(dev)
    ids, tw = fes[0].route(logits, cfg.top_k, True)
    for i in range(7):  # the last call reads weights that are not in any cache
        fes[i % 3].apply(A, ids, tw)
    torch.cuda.synchronize()
    stamps = np.zeros((STAGES, WORKGROUPS, SLOTS), dtype=np.uint64)
    rc = lib.vk_debug_decode_trace(stamps.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise SystemExit(f"vk_debug_decode_trace: HIP error {rc}")

    for stage in range(STAGES):
        t = stamps[stage].astype(np.int64)
        t = t[t[:, 4] > t[:, 0]]  # workgroups that had a slice
        if len(t) == 0:
            print(f"{args.workload} stage {stage}: the decode kernel did not run")
            continue
        first = t[:, 0].min()
        print(f"{args.workload} stage {stage}: {len(t)} workgroups, first entry -> last end "
              f"{(t[:, 4].max() - first) / 100.0:.1f} us, entries within {(t[:, 0].max() - first) / 100.0:.1f} us")
        for label, a, b in PHASES:
            d = (t[:, b] - t[:, a]) / 100.0
            print(f"  {label:44s} mean {d.mean():6.2f}  min {d.min():6.2f}  max {d.max():6.2f}")


if __name__ == "__main__":
    main()
