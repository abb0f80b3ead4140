"""Where the native library is looked for.

The search order is the reference loader's contract
(src/python/vkernels/native_runtime.py:10-26): an explicit VKERNELS_LIB path wins and
must exist; otherwise the first hit among the package directory,
$VKERNELS_BUILD_DIR/src/c and $K3/home/pylib.
"""
from __future__ import annotations

import os
from pathlib import Path

# (environment variable or None for the package directory, sub-path below it)
_SEARCH_ROOTS = ((None, ()), ("VKERNELS_BUILD_DIR", ("src", "c")), ("K3", ("home", "pylib")))


def search_directories() -> list[Path]:
    """The directories that exist in the environment's terms, in search order."""
    found = []
    for variable, below in _SEARCH_ROOTS:
        root = Path(__file__).parent if variable is None else os.environ.get(variable)
        if root:
            found.append(Path(root).joinpath(*below))
    return found


def find_library(names=("libvkernels_hip.so",)) -> str | None:
    explicit = os.environ.get("VKERNELS_LIB")
    if explicit:  # a missing file here is an error (FileNotFoundError), not a fall-through
        return str(Path(explicit).expanduser().resolve(strict=True))
    hits = (d / n for d in search_directories() for n in names)
    return next((str(p.resolve()) for p in hits if p.is_file()), None)
