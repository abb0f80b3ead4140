"""Compile libvkernels_hip.so for gfx950 with hipcc, in-tree.

    python -m vkernels_amd.build

hipcc cross-compiles without a GPU.  The library lands next to this file,
where the loader looks first.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB = PKG / "libvkernels_hip.so"

SOURCES = ["moe_route.hip", "moe_align.hip", "moe_dequant.hip", "moe_gemm.hip", "hip_capi.cpp"]

# -packed-fp32-ops off: hipcc must not form packed fp32 arithmetic.
# No fast-math: the router relies on IEEE division and un-contracted arithmetic.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-lto",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> Path:
    cmd = [hipcc(), *FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-x", "hip",
           *[str(CSRC / s) for s in SOURCES], "-o", str(LIB)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
