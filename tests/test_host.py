"""CPU tests of the host side: the Python helpers that mirror the reference's
`vllm_experts` module for this path (cases modelled on the reference's
tests/python/test_vllm_experts.py), the loader rules, and the C ABI library
itself -- that it loads without a GPU, exports every symbol the header
declares and rejects contract violations before touching a device."""
from __future__ import annotations

import ctypes
import os
import re
import tempfile
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import native_runtime
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

ROOT = Path(__file__).resolve().parent.parent


# ---- pure helpers -------------------------------------------------------------

def test_max_em_count_pads_to_64():
    # reference: tests/python/test_vllm_experts.py:54-59
    assert ve.max_em_count(1, 16, 896) == ((16 + 896 + 63) // 64) * 64
    assert ve.max_em_count(8192, 16, 896) % 64 == 0
    assert ve.max_em_count(0, 1, 0) == 0


def test_max_num_tokens_hint_env(monkeypatch):
    # reference: tests/python/test_vllm_experts.py:61-96
    for k in ("MAX_NUM_BATCHED_TOKENS", "VLLM_MAX_NUM_BATCHED_TOKENS"):
        monkeypatch.delenv(k, raising=False)
    assert ve.max_num_tokens_hint() == 8192
    monkeypatch.setenv("MAX_NUM_BATCHED_TOKENS", "12345")
    assert ve.max_num_tokens_hint() == 12345
    monkeypatch.setenv("MAX_NUM_BATCHED_TOKENS", "not-a-number")
    assert ve.max_num_tokens_hint() == 8192


def test_default_block_size():
    assert ve.default_block_size(1) == 16 and ve.default_block_size(32) == 16
    assert ve.default_block_size(33) == 64 and ve.default_block_size(8192) == 64
    # with top_k: by routed rows, as the library splits its kernels
    assert ve.default_block_size(64, 4) == 16 and ve.default_block_size(128, 4) == 16
    assert ve.default_block_size(129, 4) == 128 and ve.default_block_size(2047, 8) == 128
    assert ve.default_block_size(2048, 8) == 128 and ve.default_block_size(16384, 8) == 128
    # a caller that gives the prepacked weights: blocks of 16 while the first stage's kernel
    # can align for itself (256 routed rows), then blocks of 32 (a block a pass on the chunked
    # decode kernel) up to 28 rows per expert, as long as the runs fit the kernels' list of 512
    c4 = dict(packed_experts=64, hidden=4096, ispp=1536)
    assert ve.default_block_size(42, 6, **c4) == 16 and ve.default_block_size(43, 6, **c4) == 32      # 252 / 258 rows
    assert ve.default_block_size(298, 6, **c4) == 32 and ve.default_block_size(299, 6, **c4) == 128   # 1788 / 1794 rows
    c2 = dict(packed_experts=128, hidden=2880, ispp=2880)
    assert ve.default_block_size(64, 4, **c2) == 16 and ve.default_block_size(896, 4, **c2) == 32
    assert ve.default_block_size(897, 4, **c2) == 128
    assert ve.default_block_size(128, 4, packed_experts=8, hidden=2880, ispp=2880) == 32   # 512 rows: decode-sized anyway
    assert ve.default_block_size(129, 4, packed_experts=8, hidden=2880, ispp=2880) == 128
    assert ve.default_block_size(250, 8, packed_experts=256, hidden=7168, ispp=2048) == 32   # rows of any K
    assert ve.default_block_size(512, 8, packed_experts=500, hidden=2880, ispp=2880) == 128   # room for 12 runs only
    lib = ve.load_libvkernels_hip()
    assert lib.vk_hip_moe_decode_max_rows(0, 16) == 512 and lib.vk_hip_moe_decode_max_rows(64, 16) == 576
    assert lib.vk_hip_moe_decode_max_rows(64, 32) == 1792 and lib.vk_hip_moe_decode_max_rows(0, 32) == 0
    assert lib.vk_hip_moe_decode_max_rows(64, 128) == 512


@pytest.mark.parametrize("M,top_k,E,bs", [(1, 1, 8, 16), (4, 2, 8, 16), (64, 4, 32, 64),
                                          (100, 8, 256, 64), (7, 6, 64, 32)])
def test_align_with_map_matches_oracle(M, top_k, E, bs):
    """No map, identity map and a skipping map against the oracle's alignment
    (reference: tests/python/test_vllm_experts.py:104-175)."""
    rng = np.random.default_rng(M * 131 + E)
    ids = rng.integers(0, E, size=M * top_k).astype(np.int32)
    ident = np.arange(E, dtype=np.int32)
    skip = np.full(E, -1, dtype=np.int32)
    owned = rng.permutation(E)[:max(1, E // 4)]
    skip[owned] = np.arange(owned.size, dtype=np.int32)
    for emap, local_n in ((None, E), (ident, E), (skip, owned.size)):
        s, e, em = ve.moe_align_block_size_with_map(ids, E, bs, emap)
        rs, re_, rem = oracle.moe_align_block_size_with_map(ids, E, bs, emap, local_n=local_n)
        assert int(em) == rem
        assert np.array_equal(np.asarray(s)[:rem], rs[:rem])
        assert np.array_equal(np.asarray(e)[:rem // bs], re_[:rem // bs])


def test_align_with_map_empty_routing_keeps_one_block():
    # reference: tests/python/test_vllm_experts.py:159-175
    ids = np.zeros(4, dtype=np.int32)
    emap = np.array([-1, -1], dtype=np.int32)
    s, e, em = ve.moe_align_block_size_with_map(ids, 2, 16, emap)
    assert int(em) >= 16 and np.all(np.asarray(e)[:int(em) // 16] < 0)


@pytest.mark.parametrize("kind", ["uniform", "hot", "skewed", "tp_shard", "empty"])
def test_align_em_bound_covers_actual(kind):
    """_align_em_bound is an upper bound of the EM the alignment produces
    (reference: tests/python/test_vllm_experts.py:230-275)."""
    rng = np.random.default_rng(5)
    E, top_k, bs, M = 64, 6, 64, 300
    ids = rng.integers(0, E, size=M * top_k).astype(np.int32)
    emap, local_n = None, E
    if kind == "hot":
        ids[:] = 3
    if kind == "skewed":
        ids = np.minimum((rng.pareto(1.1, M * top_k) * 2).astype(np.int32), E - 1)
    if kind == "tp_shard":
        local_n = 16
        emap = np.full(E, -1, dtype=np.int32)
        emap[16:32] = np.arange(16, dtype=np.int32)
    if kind == "empty":
        local_n = 1
        emap = np.full(E, -1, dtype=np.int32)
    _, _, em = oracle.moe_align_block_size_with_map(ids, E, bs, emap, local_n=local_n)
    bound = ve._align_em_bound(M, top_k, local_n, bs)
    assert em <= bound and bound % bs == 0 and bound >= bs
    assert bound == oracle.align_em_bound(M, top_k, local_n, bs)


# ---- CaptureSafeScratch (reference: tests/python/test_vllm_experts.py:318-405) --

def _cpu():
    return torch.device("cpu")


def test_scratch_allocates_once_at_capacity():
    s = ve.CaptureSafeScratch()
    a = s.get("out", 10, dtype=torch.float32, device=_cpu(), capacity=100)
    assert a.numel() == 10
    b = s.get("out", 60, dtype=torch.float32, device=_cpu())
    assert b.numel() == 60 and a.data_ptr() == b.data_ptr()
    c = s.get("other", 5, dtype=torch.float32, device=_cpu())
    assert c.data_ptr() != a.data_ptr()
    assert len(s.keys()) == 2
    s.reset()
    assert s.keys() == []


def test_scratch_growth_refused_during_capture_only():
    capturing = {"on": True}
    s = ve.CaptureSafeScratch(capture_probe=lambda: capturing["on"])
    capturing["on"] = False
    s.get("act", 8, dtype=torch.float32, device=_cpu(), capacity=16)
    capturing["on"] = True
    assert s.get("act", 16, dtype=torch.float32, device=_cpu()).numel() == 16  # within capacity
    with pytest.raises(RuntimeError):
        s.get("act", 17, dtype=torch.float32, device=_cpu(), name="act_scratch")
    capturing["on"] = False
    assert s.get("act", 17, dtype=torch.float32, device=_cpu()).numel() == 17


def test_scratch_negative_count():
    with pytest.raises(ValueError):
        ve.CaptureSafeScratch().get("x", -1, dtype=torch.float32, device=_cpu())


# ---- loader (reference: native_runtime.py:10-26, tests/python/test_vllm_experts.py:281-310)

def test_loader_prefers_vkernels_lib(monkeypatch):
    with tempfile.TemporaryDirectory() as d:
        lib = os.path.join(d, "libvkernels_hip.so")
        Path(lib).write_bytes(b"\x7fELF")
        monkeypatch.setenv("VKERNELS_LIB", lib)
        assert native_runtime.find_library(("libvkernels_hip.so",)) == str(Path(lib).resolve())
        assert ve.find_libvkernels_hip() == str(Path(lib).resolve())


def test_loader_missing_override_is_an_error(monkeypatch):
    # as in the reference: an override that does not exist is not silently skipped
    monkeypatch.setenv("VKERNELS_LIB", "/definitely/not/here/libvkernels_hip.so")
    with pytest.raises(FileNotFoundError):
        ve.find_libvkernels_hip()


def test_loader_search_order(monkeypatch):
    for k in ("VKERNELS_LIB", "VKERNELS_BUILD_DIR", "K3"):
        monkeypatch.delenv(k, raising=False)
    assert native_runtime.find_library(("libvkernels_nope.so",)) is None
    with tempfile.TemporaryDirectory() as d:
        (Path(d) / "src" / "c").mkdir(parents=True)
        (Path(d) / "home" / "pylib").mkdir(parents=True)
        (Path(d) / "home" / "pylib" / "libvkernels_nope.so").write_bytes(b"\x7fELF")
        monkeypatch.setenv("K3", d)
        assert native_runtime.find_library(("libvkernels_nope.so",)).endswith("home/pylib/libvkernels_nope.so")
        (Path(d) / "src" / "c" / "libvkernels_nope.so").write_bytes(b"\x7fELF")
        monkeypatch.setenv("VKERNELS_BUILD_DIR", d)
        assert native_runtime.find_library(("libvkernels_nope.so",)).endswith("src/c/libvkernels_nope.so")
    built = ROOT / "vkernels_amd" / "libvkernels_hip.so"
    if built.exists():  # the package directory comes first
        assert ve.find_libvkernels_hip() == str(built.resolve())


# ---- the C ABI library ------------------------------------------------------------

@pytest.fixture(scope="module")
def lib():
    path = ROOT / "vkernels_amd" / "libvkernels_hip.so"
    if not path.exists():
        pytest.skip("libvkernels_hip.so is not built (python -m vkernels_amd.build)")
    return ctypes.CDLL(str(path))


def _declared_symbols():
    text = (ROOT / "include" / "vkernels_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vk_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared_symbols()
    assert len(names) >= 14 and "vk_hip_fused_moe_mxfp4" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/vkernels_hip.h but not exported: {missing}"


def test_version_and_error_plumbing(lib):
    lib.vk_version.restype = ctypes.c_char_p
    lib.vk_last_error.restype = ctypes.c_char_p
    assert lib.vk_version()
    assert lib.vk_has_cuda() == 0
    lib.vk_set_last_error(0, b"")
    assert lib.vk_last_error_code() == 0 and lib.vk_last_error() == b""
    lib.vk_set_last_error(3, b"boom")
    assert lib.vk_last_error_code() == 3 and lib.vk_last_error() == b"boom"
    lib.vk_set_last_error(0, b"")


def test_max_em_matches_oracle(lib):
    lib.vk_moe_align_block_size_max_em.restype = ctypes.c_size_t
    lib.vk_moe_align_block_size_max_em.argtypes = [ctypes.c_int] * 4
    for M, k, bs, E in [(1, 1, 16, 8), (64, 4, 64, 32), (8192, 8, 64, 256), (0, 2, 16, 4),
                        (33, 6, 32, 64)]:
        assert lib.vk_moe_align_block_size_max_em(M, k, bs, E) == oracle.align_max_em(M, k, bs, E)


def test_workspace_bytes(lib):
    f = lib.vk_hip_fused_moe_mxfp4_workspace_bytes
    f.restype = ctypes.c_size_t
    f.argtypes = [ctypes.c_int] * 5
    assert f(0, 2880, 2880, 4, 64) == 0 and f(64, 2880, 2880, 4, 0) == 0
    M, H, I, k, EM = 4096, 7168, 2048, 8, 49152
    need = f(M, H, I, k, EM)
    # enough for either path.  Raw weights: both split copies (2 bytes per value) and their
    # scale rows; prepacked weights: three planes of a byte per value and a flag byte per
    # row; either way the second stage's fp32 rows and the position of every flat index
    raw = 2 * M * H + M * H // 32 + 2 * EM * I + EM * I // 32 + 4 * EM * H + 4 * M * k
    packed = 3 * M * H + 3 * EM * I + M + EM + 4 * EM * H + 4 * M * k
    floor = max(raw, packed)
    assert floor <= need <= floor + M * 16 + EM * 16 + 6 * 256
    assert f(M + 1, H, I, k, EM) > need and f(M, H, I, k, EM + 64) > need
    # rows are padded to whole K steps of 128
    assert f(64, 2880, 2880, 4, 512) >= 3 * 64 * 2944 + 3 * 512 * 2944


def test_entry_points_reject_contract_violations_without_a_device(lib):
    """Argument checks run before any launch, so they can be exercised on a machine
    without a GPU: the int-returning calls report the code, the void ones leave it in
    vk_last_error."""
    lib.vk_last_error.restype = ctypes.c_char_p
    P = ctypes.c_void_p
    align = lib.vk_hip_moe_align_block_size
    align.restype = ctypes.c_int
    align.argtypes = [P, P] + [ctypes.c_int] * 6 + [P] * 4
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, P)
    assert align(None, None, 4, 2, 16, 8, 8, 64, p, p, p, None) != 0          # null topk_ids
    assert align(p, None, 4, 2, 24, 8, 8, 64, p, p, p, None) != 0             # block size not /16
    assert align(p, None, 4, 2, 16, 8, 8, 8, p, p, p, None) != 0              # max_EM too small
    assert lib.vk_last_error_code() != 0 and lib.vk_last_error() != b""
    route = lib.vk_hip_moe_route_topk
    route.restype = ctypes.c_int
    route.argtypes = [P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, P, P, P]
    assert route(p, 4, 8, 9, 1, p, p, None) != 0                              # top_k > experts
    assert route(None, 4, 8, 2, 1, p, p, None) != 0
    moe = lib.vk_hip_fused_moe_mxfp4
    moe.restype = None
    moe.argtypes = ve._MOE_ARGTYPES
    lib.vk_set_last_error(0, b"")
    F = ctypes.c_float
    moe(p, p, p, p, p, p, p, p, p, 4, 100, 128, 2, p, p, 64, F(0), 0, F(4), F(25), None, None,
        16, None)                                                             # hidden not /64
    assert lib.vk_last_error_code() != 0 and b"vk_hip_fused_moe_mxfp4" in lib.vk_last_error()
    lib.vk_set_last_error(0, b"")
    odd = P(ctypes.addressof(buf) + 2)
    moe(p, p, p, p, p, p, p, p, p, 4, 128, 128, 2, p, p, 64, F(0), 0, F(4), F(25), odd, None,
        16, None)                                                             # bias not aligned like a float
    assert lib.vk_last_error_code() != 0 and b"aligned" in lib.vk_last_error()
    lib.vk_set_last_error(0, b"")
    moe(p, p, p, p, p, p, p, p, p, 0, 128, 128, 2, p, p, 64, F(0), 0, F(4), F(25), None, None,
        16, None)                                                             # nothing routed: no-op
    assert lib.vk_last_error_code() == 0


# ---- synthetic inputs ------------------------------------------------------------------

def test_synth_is_deterministic_and_prefix_stable():
    a = synth.make_activations(8, 64, 11)
    b = synth.make_activations(16, 64, 11)
    assert np.array_equal(a, b[:8])  # a shorter batch is a prefix of a longer one
    w1 = synth.make_weights(2, 64, 64, 5)
    w2 = synth.make_weights(2, 64, 64, 5)
    assert torch.equal(w1.w13, w2.w13) and torch.equal(w1.w2_scale, w2.w2_scale)
    codes = torch.cat([w1.w13.flatten() & 15, w1.w13.flatten() >> 4])
    assert set(codes.tolist()) <= set(synth.FINITE_CODES)
    assert int(w1.w13_scale.min()) >= 123 and int(w1.w13_scale.max()) <= 129
    lg = synth.make_logits("zipf", 512, 128, 3)
    top = np.bincount(np.argsort(-lg, axis=1)[:, :4].ravel(), minlength=128)
    assert top.max() > 6 * np.median(top)


# ---- launch-shape heuristics and the tuning store (reference: kernels/common/heuristics.hpp:20-61,
# core/tuning.hpp:11-25; tests/core/test_tuning.cpp reads the same format) ----
def test_tile_candidates_and_compiled_in_rules():
    for stage in (0, 1):
        cands = ve.moe_tile_candidates(stage)
        assert len(cands) == 10 and len(set(cands)) == 10
        assert sum(c[0] == 4 for c in cands) == 2         # the chunked decode kernel (prepacked form)
        plain = {c[1:] for c in cands if c[0] == 2}
        assert all(c[1:] in plain for c in cands if c[0] == 3)   # a K-split shape has its plain form to fall back to
        assert (0, 4, 4, 0) in cands                      # the tile kernels
        for n_flat, K, ncols in [(1, 2880, 2880), (256, 2880, 2880), (512, 7168, 2048), (513, 2880, 2880),
                                 (131072, 7168, 2048), (64, 256, 512)]:
            shape, stored = ve.moe_tile_query(stage, K, ncols, n_flat)
            assert not stored and shape in cands, (stage, n_flat, shape)   # selectors return table entries only
            # the decode kernels up to 512 routed rows, where a pass's rows fit LDS and registers
            assert (shape[0] in (2, 3)) == (n_flat <= 512 and K <= (4096 if stage == 0 else 3072))
    assert ve.moe_tile_query(0, 2880, 2880, 128)[0] == (2, 8, 2, 2) and ve.moe_tile_query(1, 2880, 2880, 128)[0] == (2, 8, 1, 4)
    assert ve.moe_tile_query(0, 4096, 1536, 6)[0] == (2, 4, 2, 8)                   # rows of K = 4096
    # ... which the kernels on the prepacked form take with 8 wavefronts (and K shared for one token)
    assert ve.moe_tile_query(0, 4096, 1536, 198, packed=True)[0] == (2, 8, 2, 2)
    assert ve.moe_tile_query(0, 4096, 1536, 6, packed=True)[0] == (3, 8, 2, 4)
    assert ve.moe_tile_query(0, 2880, 2880, 256, packed=True)[0] == ve.moe_tile_query(0, 2880, 2880, 256)[0]
    # the chunked kernel: rows of a K beyond those, and every call in blocks of 32 (prepacked form only)
    assert ve.moe_tile_query(0, 7168, 2048, 64, packed=True)[0] == (4, 8, 2, 4)
    assert ve.moe_tile_query(1, 4224, 512, 64, packed=True)[0] == (4, 8, 1, 4)
    assert ve.moe_tile_query(0, 2880, 2880, 512, packed=True, block_size=32)[0] == (4, 8, 2, 4)
    assert ve.moe_tile_query(1, 2880, 2880, 512, packed=True, block_size=32)[0] == (4, 8, 1, 4)
    assert ve.moe_tile_query(0, 7168, 2048, 64)[0] == (0, 4, 4, 0)
    # one token: fewer units than half the device's wavefronts, K shared between them
    assert ve.moe_tile_query(0, 2880, 2880, 4)[0] == (3, 8, 2, 4) and ve.moe_tile_query(1, 2880, 2880, 4)[0] == (3, 8, 1, 8)
    assert ve.moe_tile_query(1, 1536, 4096, 6)[0] == (3, 8, 2, 4)                   # ... with two tiles a unit
    assert ve.moe_tile_query(0, 2880, 2880, 8)[0] == (2, 8, 2, 2) and ve.moe_tile_query(0, 512, 2880, 4)[0] == (2, 8, 2, 2)
    assert ve.moe_tile_query(0, 256, 512, 32)[0] == (2, 8, 2, 2) and ve.moe_tile_query(1, 512, 256, 32)[0] == (2, 8, 1, 4)
    assert ve.default_block_size(0, 4) == 16 and ve.default_block_size(1 << 20, 32) == 128


def test_tuning_store_round_trip(tmp_path):
    lib = ve.load_libvkernels_hip()
    key = (0, 2880, 2880, 200)
    before, _ = ve.moe_tile_query(*key)
    other = next(c for c in ve.moe_tile_candidates(0)
                 if c != before and c[0] == 2 and c not in ve.moe_tile_candidates(1))   # a stage-0 shape only
    try:
        ve.moe_tile_set(*key, other)
        assert ve.moe_tile_query(*key) == (other, True)
        assert ve.moe_tile_query(0, 2880, 2880, 129) == (other, True)      # same bucket of 256 rows
        assert ve.moe_tile_query(0, 2880, 2880, 128)[1] is False           # the next bucket down
        assert ve.moe_tile_query(1, 2880, 2880, 200)[1] is False
        with pytest.raises(ValueError):
            ve.moe_tile_set(*key, (2, 8, 3, 4))                            # not a compiled shape
        with pytest.raises(ValueError):
            ve.moe_tile_set(1, 2880, 2880, 200, other)                     # a stage-0 shape for stage 1
        text = ve.moe_tuning_dump()
        assert text.startswith("# vk-native-tuning/2\n") and "key=0,2880,2880,256\n" in text
        (tmp_path / "moe_fused.gfx950.tune").write_text(
            text.replace("key=0,2880,2880,256", "key=0,4096,1536,64")
            + "garbage line\nkey=1,4096\nwaves=8\n"                          # malformed key: skipped
            + "key=1,1536,4096,64\nvariant=2\nwaves=8\nnt=7\ndepth=4\n"      # not compiled: skipped
            + "key=1,1536,4096,512\nvariant=2\nwaves=8\nnt=1\n"              # incomplete: skipped
            + "# comment\n\nkey=1,1536,4096,32\nvariant=2\nwaves=8\nnt=1\ndepth=12\n")
        assert ve.moe_tuning_load(str(tmp_path)) == 2
        assert ve.moe_tile_query(0, 4096, 1536, 40) == (other, True)
        assert ve.moe_tile_query(1, 1536, 4096, 17) == ((2, 8, 1, 12), True)
        assert ve.moe_tile_query(1, 1536, 4096, 64)[1] is False and ve.moe_tile_query(1, 1536, 4096, 512)[1] is False
        assert ve.moe_tile_query(*key) == (other, True)                    # a record set by hand survives a load
        assert ve.moe_tuning_load(str(tmp_path / "nowhere")) == 0          # no file: the file's records go
        assert ve.moe_tile_query(1, 1536, 4096, 17)[1] is False
        # a body without the format's first line, or swept on another architecture, is no
        # store of this library's: its records are not taken (and the last load's go)
        good = (tmp_path / "moe_fused.gfx950.tune").read_text()
        assert ve.moe_tuning_load(str(tmp_path)) == 2
        (tmp_path / "moe_fused.gfx950.tune").write_text(good.split("\n", 1)[1])
        assert ve.moe_tuning_load(str(tmp_path)) == 0 and ve.moe_tile_query(1, 1536, 4096, 17)[1] is False
        (tmp_path / "moe_fused.gfx950.tune").write_text(good.replace("arch=gfx950", "arch=gfx942"))
        assert ve.moe_tuning_load(str(tmp_path)) == 0 and ve.moe_tile_query(1, 1536, 4096, 17)[1] is False
        (tmp_path / "moe_fused.gfx950.tune").write_text(good.replace("# arch=gfx950", "# swept"))
        assert ve.moe_tuning_load(str(tmp_path)) == 2                      # no arch named: the file name's
    finally:
        ve.moe_tile_set(*key, None)
        ve.moe_tuning_load(str(tmp_path / "nowhere"))
    assert ve.moe_tile_query(*key) == (before, False)
    assert lib.vk_hip_moe_tile_set(2, 64, 64, 1, None) == ve.VK_ERROR_INVALID_ARGUMENT


def test_stage_entry_points_reject_contract_violations_without_a_device():
    """The four stages of the tensor-parallel split validate on the host and launch
    nothing for a refused or an empty call."""
    lib = ve.load_libvkernels_hip()
    P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    gu = lib.vk_hip_moe_gateup_preact
    gu.restype, gu.argtypes = I, [P] * 6 + [I] * 8 + [P]
    dn = lib.vk_hip_moe_down_preact
    dn.restype, dn.argtypes = I, [P] * 6 + [I] * 8 + [P]
    ep = lib.vk_hip_moe_act_epilogue
    ep.restype, ep.argtypes = I, [P] * 5 + [I] * 4 + [F, I, F, F, I, P]
    cb = lib.vk_hip_moe_combine
    cb.restype, cb.argtypes = I, [P] * 6 + [I] * 5 + [P, ctypes.c_size_t, P]
    bad = ve.VK_ERROR_INVALID_ARGUMENT
    nil = (None,) * 6
    #                         M  hidden ispp k  EM  k_base k_dim bs
    assert gu(*nil, 0, 256, 512, 2, 0, 0, 256, 16, None) == 0             # nothing routed
    assert gu(*nil, 4, 256, 512, 2, 32, 0, 256, 16, None) == bad          # null buffers
    assert "null" in ve.last_error(lib)
    assert gu(*nil, 4, 256, 512, 2, 32, 4, 128, 16, None) == bad          # k_base not a multiple of 8
    assert gu(*nil, 4, 256, 512, 2, 32, 0, 96, 16, None) == bad           # slice not a multiple of 64
    assert gu(*nil, 4, 256, 512, 2, 32, 192, 128, 16, None) == bad        # slice past the row
    assert gu(*nil, 4, 256, 512, 2, 32, 0, 256, 24, None) == bad          # block size
    assert gu(*nil, 4, 256, 512, 0, 32, 0, 256, 16, None) == bad          # top_k
    assert dn(*nil, 4, 512, 256, 2, 32, 0, 512, 16, None) == bad
    assert dn(*nil, 4, 512, 250, 2, 32, 0, 512, 16, None) == bad          # output width
    assert dn(*nil, 0, 512, 256, 2, 0, 0, 512, 16, None) == 0
    assert ep(None, None, None, None, None, 4, 2, 32, 512, 0.0, 0, 4.0, 25.0, 16, None) == bad
    assert ep(None, None, None, None, None, 4, 2, 32, 512, 0.0, 5, 4.0, 25.0, 16, None) == bad   # activation
    assert ep(None, None, None, None, None, 0, 2, 0, 512, 0.0, 0, 4.0, 25.0, 16, None) == 0
    assert cb(*nil, 4, 256, 2, 32, 16, None, 0, None) == bad
    assert cb(*nil, 4, 254, 2, 32, 16, None, 0, None) == bad
    assert cb(*nil, 0, 256, 2, 0, 16, None, 0, None) == 0
