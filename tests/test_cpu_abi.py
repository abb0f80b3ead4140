"""The host-side C ABI of the path (include/vkernels_cpu.h), as a C consumer sees it.

The header declares the reference's CPU entry points for the path
(src/c/vkernels/capi/capi.hpp:470-539); in this repository the CPU checker serves them.
A C program that includes nothing but that header is compiled, linked against
oracle/liboracle.so and run: it holds the reference's own known-answer cases for the ABI
(align example, all-ones closed forms, SiTU, bias only, null guards, quantiser table,
sort, scatter).  The compiler also holds the checker's definitions to the header's
prototypes (oracle/capi_oracle.c includes it).  No GPU involved.
"""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

import oracle

ROOT = Path(__file__).resolve().parent.parent


def test_c_consumer_of_the_cpu_abi(tmp_path):
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    lib = Path(oracle.lib()._name).resolve()
    exe = tmp_path / "cpu_abi_check"
    subprocess.run([cc, "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "cpu_abi_check.c"), "-o", str(exe), f"-L{lib.parent}", "-loracle",
                    f"-Wl,-rpath,{lib.parent}", "-lm"], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "all checks held" in res.stdout


def test_every_declared_cpu_symbol_is_served_by_the_checker():
    header = (ROOT / "include" / "vkernels_cpu.h").read_text()
    declared = sorted(set(re.findall(r"\b(vk_\w+)\s*\(", header)))
    assert {"vk_fused_moe_mxfp4", "vk_moe_align_block_size", "vk_moe_align_block_size_max_em",
            "vk_mxfp4_moe_quant", "vk_mxfp4_moe_sort", "vk_mxfp4_moe_sort_scales",
            "vk_mxfp4_moe_scatter_reduce", "vk_mxfp4_moe_scatter_reduce_q"} <= set(declared)
    handle = oracle.lib()
    for name in declared:
        getattr(handle, name)   # AttributeError names a declared symbol the checker lacks


def test_both_headers_compile_together(tmp_path):
    """The device header and the host header share the status codes under one guard."""
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "both.c"
    src.write_text('#include "vkernels_hip.h"\n#include "vkernels_cpu.h"\n#include "vkernels_cpu.h"\n'
                   "int main(void) { return VK_OK; }\n")
    subprocess.run([cc, "-std=c11", "-Wall", "-Werror", f"-I{ROOT / 'include'}", "-c", str(src), "-o",
                    str(tmp_path / "both.o")], check=True)
