"""The prefill kernel's address arithmetic, checked on the CPU: the kernel forms every byte
offset through the functions of vkernels_amd/csrc/moe_prefill_layout.hpp, and
tests/prefill_layout_check.cpp (compiled here with g++) walks all lanes, K steps and tiles of
a problem with the same functions: loads inside the prepacked weights and the split rows,
copies inside their ring slot without overlap, operand reads hitting exactly the bytes of
their row, term and K block, staging areas inside the ring.  The same program also walks the
K loop's schedule of a wavefront (prologue, every group of every step, the step's one wait
and barrier, the tail, loops of one and two steps, one to four live row tiles, one to three
terms) built from the schedule functions the kernel's counted waits are built from: issued
against waited vector-memory operations, ring slots written against slots still read,
weight register sets loaded against sets still multiplied.  Shapes: every configuration of
the benchmark list, both stages, every term count, and ragged ones."""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))
from vkernels_amd import synth  # noqa: E402


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = tmp_path_factory.mktemp("layout") / "prefill_layout_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-Wall", "-Werror", f"-I{ROOT / 'vkernels_amd' / 'csrc'}",
                    str(ROOT / "tests" / "prefill_layout_check.cpp"), "-o", str(exe)], check=True)
    return exe


def _shapes():
    for name in ("c0", "c1", "c2", "c3", "c4"):
        cfg = synth.CONFIGS[name]
        T = max(cfg.Ts)
        em = T * cfg.top_k + cfg.E * 127                      # the largest padded row count
        yield name, 0, cfg.H, cfg.I, cfg.E, T                 # stage 0: rows of A
        yield name, 1, cfg.I, cfg.H, cfg.E, em                # stage 1: sorted rows of act
    yield "ragged", 0, 192, 64, 3, 5                          # one unit, K below two steps
    yield "ragged", 1, 64, 192, 3, 40                         # stage 1's last unit half empty
    yield "ragged", 0, 8128, 4032, 2, 17                      # K and ncols one block short of a multiple of 128


@pytest.mark.parametrize("terms", [1, 2, 3])
def test_every_offset_of_the_prefill_kernel(checker, terms):
    for name, stage, K, ncols, E, rows in _shapes():
        res = subprocess.run([str(checker), str(stage), str(terms), str(K), str(ncols), str(E), str(rows)],
                             capture_output=True, text=True)
        assert res.returncode == 0, f"{name} stage {stage} terms {terms}: {res.stderr.strip()}"


def test_the_checker_notices_a_wrong_layout(checker, tmp_path):
    """The walk is not vacuous: with the rotation of the row copies removed from a copy of the
    header, the operand reads no longer find their bytes."""
    src = (ROOT / "vkernels_amd" / "csrc" / "moe_prefill_layout.hpp").read_text()
    assert "16u * (uint32_t)(c ^ r)" in src
    (tmp_path / "moe_prefill_layout.hpp").write_text(src.replace("16u * (uint32_t)(c ^ r)", "16u * (uint32_t)(c)"))
    exe = tmp_path / "broken"
    subprocess.run(["g++", "-O2", "-std=c++17", f"-I{tmp_path}", str(ROOT / "tests" / "prefill_layout_check.cpp"),
                    "-o", str(exe)], check=True)
    res = subprocess.run([str(exe), "0", "3", "2880", "2880", "4", "64"], capture_output=True, text=True)
    assert res.returncode == 1 and "FAILED" in res.stderr


def test_the_checker_notices_a_wait_that_counts_wrong(tmp_path):
    """The schedule walk is not vacuous either: with the prologue's wait letting one more
    operation stay outstanding than the kernel's does, the first operand read is flagged."""
    exe = tmp_path / "broken_wait"
    subprocess.run(["g++", "-O2", "-std=c++17", "-DVK_LAYOUT_BREAK_WAIT", f"-I{ROOT / 'vkernels_amd' / 'csrc'}",
                    str(ROOT / "tests" / "prefill_layout_check.cpp"), "-o", str(exe)], check=True)
    res = subprocess.run([str(exe), "1", "2", "2048", "7168", "4", "640"], capture_output=True, text=True)
    assert res.returncode == 1 and "before every wavefront's copies of it have landed" in res.stderr
