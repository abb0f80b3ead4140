"""Compile libvkernels_hip.so for gfx950 with hipcc, in-tree.

    python -m vkernels_amd.build [--changed]

hipcc cross-compiles without a GPU.  The library lands next to this file,
where the loader looks first.  Every translation unit is compiled to an
object file under ``vkernels_amd/build/`` (in parallel) and the objects are
linked; ``--changed`` recompiles only the units whose sources are newer than
their object (a developer convenience: ``build()`` itself always compiles
everything).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
OBJ = PKG / "build"
LIB = PKG / "libvkernels_hip.so"

SOURCES = ["moe_route.hip", "moe_align.hip", "moe_dequant.hip", "moe_gemm.hip", "moe_prefill.hip", "static_scratch.hip",
           "moe_tuning.cpp", "moe_stages.hip",
           "hip_capi.cpp"]

# -packed-fp32-ops off: hipcc must not form packed fp32 arithmetic.
# No fast-math: the router relies on IEEE division and un-contracted arithmetic.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-lto",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def _stale(src: Path, obj: Path) -> bool:
    if not obj.is_file():
        return True
    deps = [src, *CSRC.glob("*.hpp"), *INCLUDE.glob("*.h")]
    return any(d.stat().st_mtime > obj.stat().st_mtime for d in deps)


def build(verbose: bool = False, only_changed: bool = False, out_dir: Path | None = None,
          defines: tuple[str, ...] = ()) -> Path:
    """Compiles every translation unit and links libvkernels_hip.so in the package
    directory.  With out_dir the objects and the library go there instead (a build with
    extra -D defines, say the profiling build, beside the product build, not over it)."""
    cc = hipcc()
    obj_dir = OBJ if out_dir is None else Path(out_dir) / "obj"
    lib = LIB if out_dir is None else Path(out_dir) / LIB.name
    obj_dir.mkdir(parents=True, exist_ok=True)
    jobs = []
    objects = []
    for name in SOURCES:
        src, obj = CSRC / name, obj_dir / (Path(name).stem + ".o")
        objects.append(str(obj))
        if only_changed and not _stale(src, obj):
            continue
        jobs.append([cc, *FLAGS, *(f"-D{d}" for d in defines), f"-I{INCLUDE}", f"-I{CSRC}", "-x", "hip",
                     "-c", str(src), "-o", str(obj)])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
    _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-lto", *objects, "-o", str(lib)],
         verbose)
    return lib


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="build libvkernels_hip.so for gfx950")
    ap.add_argument("--changed", action="store_true", help="recompile only what is older than its sources")
    ap.add_argument("--out", default=None, help="directory for the objects and the library (default: in tree)")
    ap.add_argument("--define", action="append", default=[], help="extra -D for every translation unit")
    ap.add_argument("--quiet", action="store_true")
    a = ap.parse_args()
    print(build(verbose=not a.quiet, only_changed=a.changed, out_dir=a.out, defines=tuple(a.define)))
