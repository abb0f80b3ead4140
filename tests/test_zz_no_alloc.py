"""The entry point that allocates nothing: vk_hip_fused_moe_mxfp4_static, whose
workspace is the device array the library itself holds.

Called through the C ABI and compared with vk_hip_fused_moe_mxfp4_ex given a
caller-owned workspace (the same kernels on another buffer: the workspace path
is deterministic, so the outputs must be bit-identical), on two calls in a row,
the second with a smaller batch -- the array then still holds the first call's
split rows, stored rows and positions.  The first call's result is also held
against the CPU oracle.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

from gpu_util import MAX_ABS_TOL, REL_L2_TOL, cpu_layer, dev, error_metrics, to_dev

pytestmark = pytest.mark.gpu

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


def _static_fn(lib):
    fn = lib.vk_hip_fused_moe_mxfp4_static
    fn.restype = _I
    fn.argtypes = [_P] * 9 + [_I] * 4 + [_P, _P, _I, _F, _I, _F, _F, _P, _P, _I, ctypes.c_uint, _P]
    return fn


def _call_both(fe, static_fn, A_bits, lg, cfg, bs):
    """(out of the static entry point, out of the _ex entry point with a caller's
    workspace, routing) for one batch.  Every buffer is allocated before the two calls."""
    T = A_bits.shape[0]
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    sids, eids, _, max_em = fe.align(ids, bs)
    act = torch.zeros(max_em * cfg.I, dtype=torch.bfloat16, device=dev())
    out_static = torch.full((T, cfg.H), float("nan"), dtype=torch.float32, device=dev())
    out_ex = torch.full((T, cfg.H), float("nan"), dtype=torch.float32, device=dev())
    need = int(fe.ws_bytes_fn(T, cfg.H, cfg.I, cfg.top_k, max_em))
    assert 0 < need <= int(fe.lib.vk_hip_static_scratch_bytes())
    ws = torch.empty(need, dtype=torch.uint8, device=dev())
    args = (A.data_ptr(), fe.w13.data_ptr(), fe.w13_scale.data_ptr(), fe.w2.data_ptr(),
            fe.w2_scale.data_ptr(), ids.data_ptr(), tw.data_ptr(), act.data_ptr())
    tail = (T, cfg.H, cfg.I, cfg.top_k, sids.data_ptr(), eids.data_ptr(), max_em, 0.0, 0, 4.0, 25.0,
            None, None, bs)
    torch.cuda.synchronize()
    # (a first call, so that what the runtime itself sets up once per kernel -- code
    # objects, the spill area of a kernel's first dispatch -- is not taken for the entry
    # point's doing)
    assert static_fn(*args, out_static.data_ptr(), *tail, ve.MOE_OVERWRITE_OUT, None) == 0, ve.last_error(fe.lib)
    torch.cuda.synchronize()
    out_static.fill_(float("nan"))
    torch.cuda.synchronize()
    # the headline property: the call takes no device memory, from torch's allocator or
    # from the runtime (free memory of the device as the driver reports it)
    held = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    free_before = torch.cuda.mem_get_info()[0]
    st = static_fn(*args, out_static.data_ptr(), *tail, ve.MOE_OVERWRITE_OUT, None)
    assert st == 0, ve.last_error(fe.lib)
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == held
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the device's free memory"
    fe.moe_ex_fn(*args, out_ex.data_ptr(), *tail, ws.data_ptr(), need, ve.MOE_OVERWRITE_OUT, None)
    torch.cuda.synchronize()
    return out_static.cpu().numpy(), out_ex.cpu().numpy(), ids.cpu().numpy(), tw.cpu().numpy()


def test_static_scratch_entry_point_matches_the_workspace_one(hip_lib):
    fe_lib = hip_lib
    fe_lib.vk_hip_static_scratch_bytes.restype = ctypes.c_size_t
    assert fe_lib.vk_hip_static_scratch_bytes() == 64 << 20
    fe_lib.vk_hip_init.restype = _I
    assert fe_lib.vk_hip_init() == 0, ve.last_error(fe_lib)
    static_fn = _static_fn(fe_lib)
    cfg = synth.CONFIGS["c1"]
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, 1500, device=dev())
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
    wn = w.numpy()
    # 200 then 150 tokens (800 and 600 routed rows: the tile kernels, which use the
    # workspace), blocks of 16 rows so that the workspace stays below the array's size
    for T, seed, check_oracle in ((200, 9100, True), (150, 9101, False)):
        A_bits = synth.make_activations(T, cfg.H, seed)
        lg = synth.make_logits(cfg.logits, T, cfg.E, seed)
        got, ref, ids, tw = _call_both(fe, static_fn, A_bits, lg, cfg, 16)
        assert np.all(np.isfinite(got))
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
            f"T={T}: the static-scratch call differs from the workspace call"
        if check_oracle:
            rows = np.sort(np.random.default_rng(seed).choice(T, 24, replace=False))
            c = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16)
            max_rel, rel_l2, nf = error_metrics(got[rows], c["out"])
            assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (max_rel, rel_l2)


def test_static_scratch_entry_point_under_graph_capture(hip_lib):
    """What the entry point is for: captured in a HIP graph (after vk_hip_init, which
    resolves the array's address and the kernels' attributes outside the capture) and
    replayed with new activations in the same buffers; every replay is bit-identical to
    the eager call on the same inputs (the workspace path is deterministic)."""
    hip_lib.vk_hip_init.restype = _I
    assert hip_lib.vk_hip_init() == 0, ve.last_error(hip_lib)
    static_fn = _static_fn(hip_lib)
    cfg = synth.CONFIGS["c1"]
    T, bs = 160, 16
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, 1500, device=dev())
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
    A = torch.zeros((T, cfg.H), dtype=torch.bfloat16, device=dev())
    lg = to_dev(synth.make_logits(cfg.logits, T, cfg.E, 9200))
    ids, tw = fe.route(lg, cfg.top_k, True)
    sids, eids, _, max_em = fe.align(ids, bs)
    act = torch.zeros(max_em * cfg.I, dtype=torch.bfloat16, device=dev())
    out = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
    assert int(fe.ws_bytes_fn(T, cfg.H, cfg.I, cfg.top_k, max_em)) <= int(hip_lib.vk_hip_static_scratch_bytes())

    def call(stream):
        st = static_fn(A.data_ptr(), fe.w13.data_ptr(), fe.w13_scale.data_ptr(), fe.w2.data_ptr(),
                       fe.w2_scale.data_ptr(), ids.data_ptr(), tw.data_ptr(), act.data_ptr(), out.data_ptr(),
                       T, cfg.H, cfg.I, cfg.top_k, sids.data_ptr(), eids.data_ptr(), max_em, 0.0, 0, 4.0, 25.0,
                       None, None, bs, ve.MOE_OVERWRITE_OUT, ctypes.c_void_p(stream.cuda_stream))
        assert st == 0, ve.last_error(hip_lib)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(side)                                # eager warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call(side)
    for seed in (9201, 9202, 9203):
        A.copy_(to_dev(synth.make_activations(T, cfg.H, seed), torch.bfloat16))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy().copy()
        out.fill_(float("nan"))
        call(torch.cuda.current_stream())         # eager, between the replays
        torch.cuda.synchronize()
        eager = out.cpu().numpy()
        assert np.all(np.isfinite(got))
        assert np.array_equal(got.view(np.uint32), eager.view(np.uint32)), seed


def test_static_scratch_entry_point_rejects_oversize(hip_lib):
    """A prefill batch whose workspace exceeds the array: a clear error, nothing launched."""
    static_fn = _static_fn(hip_lib)
    one = torch.zeros(16, dtype=torch.int32, device=dev())
    p = one.data_ptr()
    st = static_fn(p, p, p, p, p, p, p, p, p, 4096, 7168, 2048, 8, p, p, 65536, 0.0, 0, 4.0, 25.0,
                   None, None, 128, 0, None)
    assert st == ve.VK_ERROR_OUT_OF_RANGE
    assert "bytes of scratch" in ve.last_error(hip_lib)
    torch.cuda.synchronize()
