"""Where the native library is looked for.

Same resolution order as the reference
(src/python/vkernels/native_runtime.py:10-26): the VKERNELS_LIB override, the
package directory, $VKERNELS_BUILD_DIR/src/c, $K3/home/pylib.
"""
from __future__ import annotations

import os
from pathlib import Path


def find_library(names=("libvkernels_hip.so",)) -> str | None:
    override = os.environ.get("VKERNELS_LIB")
    if override:
        return str(Path(override).expanduser().resolve(strict=True))
    locations = [Path(__file__).parent]
    build = os.environ.get("VKERNELS_BUILD_DIR")
    if build:
        locations.append(Path(build) / "src" / "c")
    k3 = os.environ.get("K3")
    if k3:
        locations.append(Path(k3) / "home" / "pylib")
    for directory in locations:
        for name in names:
            candidate = directory / name
            if candidate.is_file():
                return str(candidate.resolve())
    return None
