"""GPU checks of the contract's letter and of properties the layer must have whatever
its size: the reference harness's own error figure on a layer whose outputs are O(1),
the stage entry points against the fused call, run-to-run spread of the paths that add
with atomics and bit-identity of the ones that do not, rows behind a sentinel inside a
block, and the call sequence under HIP graph capture."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

import test_gpu_configs as cfgs
from gpu_util import (EXACT_SPLIT_MAX_ABS_TOL, EXACT_SPLIT_REL_L2_TOL, MAX_ABS_TOL, REL_L2_TOL,
                      cpu_layer, dev, error_metrics, literal_max_rel, to_dev)

pytestmark = pytest.mark.gpu

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


def _unit_scale_weights(cfg, seed):
    """Scale exponents centred on 2^-6 so that gate, up, act and the outputs are O(1)."""
    return synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev(), scale_lo=120, scale_hi=122)


@pytest.mark.parametrize("T,prepack", [(64, False), (200, False), (200, True), (700, True)])
def test_literal_reference_metric_on_unit_scale_outputs(T, prepack):
    """max |gpu - cpu| / max(|cpu|, 1) <= 2e-2, the figure of the reference's own harness
    (meta/benchmarks/test_moe_fused_correct.hip:195-214), asserted as written on a layer
    whose outputs have an RMS near 1 (where it is not below the fp32 ordering noise)."""
    cfg = synth.CONFIGS["c1"]
    seed = 5100
    w = _unit_scale_weights(cfg, seed)
    A, lg = cfgs._inputs(cfg, T, seed + T)
    kw = dict(prepack=True) if prepack else {}
    g = cfgs._run_gpu(cfg, w, A, lg, None, True, **kw)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    rms = float(np.sqrt(np.mean(c["out"].astype(np.float64) ** 2)))
    lit = literal_max_rel(g["out"], c["out"])
    max_rel, rel_l2, nf = error_metrics(g["out"], c["out"])
    print(f"c1 unit scale T={T} prepack={prepack}: rms(out)={rms:.3f} literal={lit:.3e} rel_l2={rel_l2:.3e}")
    assert 0.05 < rms < 20.0, "the case is meant to have outputs of order one"
    assert nf and lit <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL
    if not prepack:
        assert max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL


def _stage_fns(lib):
    gu = lib.vk_hip_moe_gateup_mxfp4
    gu.restype = None
    gu.argtypes = [_P] * 4 + [_I] * 4 + [_P, _P, _I, _F, _I, _F, _F, _P, _I, _P]
    dn = lib.vk_hip_moe_down_mxfp4
    dn.restype = None
    dn.argtypes = [_P] * 5 + [_I] * 4 + [_P, _P, _I, _P, _I, _P]
    return gu, dn


@pytest.mark.parametrize("T", [8, 64, 200])
def test_stage_entry_points_equal_the_fused_call(hip_lib, T):
    """vk_hip_moe_gateup_mxfp4 then vk_hip_moe_down_mxfp4 on a stream is
    vk_hip_fused_moe_mxfp4: act bit for bit, out within the spread of the atomic adds;
    and both agree with the oracle."""
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    A_bits, lg = cfgs._inputs(cfg, T, 5200 + T)
    b13 = (synth.rand_normal((cfg.E, 2 * cfg.I), 5200, 21) * 0.5).astype(np.float32)
    b2 = (synth.rand_normal((cfg.E, cfg.H), 5200, 22) * 0.5).astype(np.float32)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, b13=to_dev(b13), b2=to_dev(b2),
                         scratch=ve.CaptureSafeScratch())
    fe.use_workspace = False
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    bs = ve.default_block_size(T, cfg.top_k)
    sids, eids, _, max_em = fe.align(ids, bs)
    fused = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
    fe.fused_call(A, ids, tw, sids, eids, max_em, bs, fused)
    torch.cuda.synchronize()
    act_fused = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16,
                               device=dev()).view(torch.int16).cpu().numpy().copy()
    gu, dn = _stage_fns(hip_lib)
    act = torch.zeros(max_em * cfg.I, dtype=torch.bfloat16, device=dev())
    out = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
    gu(A.data_ptr(), fe.w13.data_ptr(), fe.w13_scale.data_ptr(), act.data_ptr(), T, cfg.H, cfg.I,
       cfg.top_k, sids.data_ptr(), eids.data_ptr(), max_em, 0.0, 0, 4.0, 25.0, fe.b13.data_ptr(), bs, None)
    dn(act.data_ptr(), fe.w2.data_ptr(), fe.w2_scale.data_ptr(), tw.data_ptr(), out.data_ptr(), T,
       cfg.H, cfg.I, cfg.top_k, sids.data_ptr(), eids.data_ptr(), max_em, fe.b2.data_ptr(), bs, None)
    torch.cuda.synchronize()
    s_np = sids.cpu().numpy()
    real = np.nonzero(s_np < T * cfg.top_k)[0]
    a0 = act_fused.reshape(max_em, cfg.I)[real]
    a1 = act.view(torch.int16).cpu().numpy().reshape(max_em, cfg.I)[real]
    assert np.array_equal(a0, a1), "the first stage alone differs from the fused call's"
    f, o = fused.cpu().numpy(), out.cpu().numpy()
    rms = float(np.sqrt(np.mean(f.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(f.astype(np.float64) - o))) <= 1e-3 * rms
    c = cpu_layer(A_bits, w.numpy(), ids.cpu().numpy(), tw.cpu().numpy(), threads=16, b13=b13, b2=b2)
    max_rel, rel_l2, nf = error_metrics(o, c["out"])
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL, (max_rel, rel_l2)


@pytest.mark.parametrize("T,use_workspace", [(64, True), (300, False), (300, True)])
def test_run_to_run_spread(T, use_workspace):
    """Paths that add into `out` with fp32 atomics (decode kernels, tile kernels without a
    workspace) may differ between runs by the order of the adds: at most 1e-3 of the RMS,
    the gate of the reference's own harness
    (meta/benchmarks/test_moe_fused_bigshape_correct.hip:250-258).  The workspace path of
    the tile kernels sums each token's rows in a fixed order: bit-identical."""
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, 5300 + T)
    outs = [cfgs._run_gpu(cfg, w, A, lg, None, use_workspace)["out"] for _ in range(3)]
    rms = float(np.sqrt(np.mean(outs[0].astype(np.float64) ** 2)))
    deterministic = use_workspace and T * cfg.top_k > 512
    for o in outs[1:]:
        if deterministic:
            assert np.array_equal(o.view(np.uint32), outs[0].view(np.uint32))
        else:
            assert float(np.max(np.abs(o.astype(np.float64) - outs[0]))) <= 1e-3 * rms


@pytest.mark.parametrize("prepack", [False, True])
def test_sentinel_inside_a_block_keeps_the_rows_behind_it(hip_lib, prepack):
    """sorted_ids entries >= M*top_k are padding wherever they stand: a caller-built
    table with a sentinel in the middle of an expert's rows must give the same layer as
    the table of the alignment kernel (workspace path and plain path)."""
    cfg = synth.CONFIGS["c1"]
    T = 200
    w = cfgs._weights(cfg, 1500)
    A_bits, lg = cfgs._inputs(cfg, T, 5400)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(),
                         prepack=prepack)
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    bs = 128
    sids, eids, _, max_em = fe.align(ids, bs)
    refs = {}
    for use_ws in (True, False):   # each path against itself (they multiply different operands)
        fe.use_workspace = use_ws
        ref = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
        fe.fused_call(A, ids, tw, sids, eids, max_em, bs, ref)
        torch.cuda.synchronize()
        refs[use_ws] = ref.cpu().numpy()
    # move every expert's rows one place down and put a sentinel at the block's first place
    # (experts with a full block keep their layout)
    s_np = sids.cpu().numpy().copy()
    n_flat = T * cfg.top_k
    moved = 0
    for b in range(max_em // bs):
        blk = s_np[b * bs:(b + 1) * bs]
        n = int(np.count_nonzero(blk < n_flat))
        if 0 < n < bs:
            blk[1:n + 1] = blk[:n].copy()
            blk[0] = n_flat
            moved += 1
    assert moved > 0
    for use_ws in (True, False):
        fe.use_workspace = use_ws
        got = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
        fe.fused_call(A, ids, tw, to_dev(s_np), eids, max_em, bs, got)
        torch.cuda.synchronize()
        m, l2, nf = error_metrics(got.cpu().numpy(), refs[use_ws])
        assert nf and l2 <= 1e-4, (use_ws, m, l2)


@pytest.mark.parametrize("T,prepack", [(1, False), (16, False), (300, False), (300, True)])
def test_call_sequence_under_graph_capture(hip_lib, T, prepack):
    """route -> align -> fused layer (out overwritten) captured in a HIP graph after an
    eager warm-up, replayed with new inputs written into the same buffers, with eager
    work between the replays: every replay equals the eager result of the same inputs
    (bit for bit on the deterministic path) and the oracle."""
    hip_lib.vk_hip_init.restype = _I
    assert hip_lib.vk_hip_init() == 0, ve.last_error(hip_lib)
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(),
                         prepack=prepack)
    A = torch.zeros((T, cfg.H), dtype=torch.bfloat16, device=dev())
    lg = torch.zeros((T, cfg.E), dtype=torch.float32, device=dev())
    out = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())

    def load(seed):
        a_bits, l_np = cfgs._inputs(cfg, T, seed)
        A.copy_(to_dev(a_bits, torch.bfloat16))
        lg.copy_(to_dev(l_np))
        return a_bits, l_np

    def run():
        ids, tw = fe.route(lg, cfg.top_k, True)
        fe.apply(A, ids, tw, out_fp32=out)
        return ids, tw

    load(5500)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # eager warm-up on the capture stream: sizes every scratch buffer
        for _ in range(2):
            run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ids_g, tw_g = run()
    deterministic = T * cfg.top_k > 512
    for seed in (5501, 5502, 5503):
        a_bits, l_np = load(seed)
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy().copy()
        ids_np, tw_np = ids_g.cpu().numpy().copy(), tw_g.cpu().numpy().copy()
        rid, rtw = oracle.route_topk(l_np, cfg.top_k, True)
        assert np.array_equal(ids_np, rid) and np.array_equal(tw_np.view(np.uint32), rtw.view(np.uint32))
        out.fill_(float("nan"))
        run()                                   # eager, between the replays
        torch.cuda.synchronize()
        eager = out.cpu().numpy().copy()
        if deterministic:
            assert np.array_equal(got.view(np.uint32), eager.view(np.uint32)), seed
        else:
            rms = float(np.sqrt(np.mean(eager.astype(np.float64) ** 2)))
            assert float(np.max(np.abs(got.astype(np.float64) - eager))) <= 1e-3 * rms, seed
        rows = np.arange(T) if T <= 64 else np.sort(np.random.default_rng(seed).choice(T, 32, replace=False))
        c = cpu_layer(a_bits[rows], w.numpy(), rid[rows], rtw[rows], threads=16)
        max_rel, rel_l2, nf = error_metrics(got[rows], c["out"])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (seed, max_rel, rel_l2)


def test_apply_hands_back_bf16_on_request(hip_lib):
    """The reference's serving class returns the layer in the activations' type
    (src/python/vkernels/vllm_experts.py:1092): output_dtype gives that, as the rounded
    fp32 result; an empty batch keeps its shape and type."""
    cfg = synth.CONFIGS["c0"]
    w = cfgs._weights(cfg, 77)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale)
    a_bits, l_np = cfgs._inputs(cfg, 16, 78)
    A = to_dev(a_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(l_np), cfg.top_k, True)
    full = fe.apply(A, ids, tw)
    half = fe.apply(A, ids, tw, output_dtype=torch.bfloat16)
    assert half.dtype == torch.bfloat16 and torch.equal(half, full.to(torch.bfloat16))
    none = fe.apply(A[:0], ids[:0], tw[:0], output_dtype=torch.bfloat16)
    assert none.dtype == torch.bfloat16 and tuple(none.shape) == (0, cfg.H)


@pytest.mark.parametrize("T,prepack,use_workspace", [(32, False, True), (300, False, False), (300, False, True),
                                                     (300, True, True)])
def test_biases_need_only_the_alignment_of_floats(hip_lib, T, prepack, use_workspace):
    """b13 / b2 that start 4 bytes into an allocation (a view inside a larger buffer), as
    the reference accepts them: the act rows are the same bits as with the 16-byte
    aligned copies, on the decode kernels, both raw-weight tile kernels and the prepacked
    path, and `out` is the same up to the spread of the atomic adds."""
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    A_bits, lg = cfgs._inputs(cfg, T, 5300 + T)
    b13 = (synth.rand_normal((cfg.E, 2 * cfg.I), 5300, 21) * 0.5).astype(np.float32)
    b2 = (synth.rand_normal((cfg.E, cfg.H), 5300, 22) * 0.5).astype(np.float32)
    res = []
    for shift in (0, 1):
        h13 = torch.zeros(b13.size + 1, dtype=torch.float32, device=dev())
        h2 = torch.zeros(b2.size + 1, dtype=torch.float32, device=dev())
        v13 = h13[shift:shift + b13.size].view(b13.shape)
        v2 = h2[shift:shift + b2.size].view(b2.shape)
        v13.copy_(to_dev(b13))
        v2.copy_(to_dev(b2))
        assert v13.data_ptr() % 16 == 4 * shift and v2.data_ptr() % 16 == 4 * shift
        fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, b13=v13, b2=v2,
                             scratch=ve.CaptureSafeScratch(), prepack=prepack)
        fe.use_workspace = use_workspace
        A = to_dev(A_bits, torch.bfloat16)
        ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
        bs = ve.default_block_size(T, cfg.top_k)
        sids, eids, _, max_em = fe.align(ids, bs)
        out = fe.apply(A, ids, tw, block_size=bs)
        torch.cuda.synchronize()
        act = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16, device=dev())
        real = np.nonzero(sids.cpu().numpy() < T * cfg.top_k)[0]
        res.append((out.cpu().numpy(), act.view(torch.int16).cpu().numpy().reshape(max_em, cfg.I)[real].copy()))
    assert np.array_equal(res[0][1], res[1][1]), "act differs with a bias that is only 4-byte aligned"
    f, o = res[0][0].astype(np.float64), res[1][0].astype(np.float64)
    rms = float(np.sqrt(np.mean(f ** 2)))
    assert float(np.max(np.abs(f - o))) <= 1e-3 * rms
