"""GPU parity of the layer as four stages (gate/up pre-activations, activation epilogue,
down pre-activations, combine) through the C ABI: each stage against the oracle's
function of the same name on the same inputs, and the tensor-parallel composition (K
slices summed between the stages) against the fused oracle.

Bars: pre-activations are fp32 sums whose order differs from the oracle's (relative to
the RMS, bounds below); the epilogue is elementwise on identical inputs (bf16 result
within one unit in the last place); the combine is the reference's sum bit for bit."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

import test_gpu_configs as cfgs
from gpu_util import EXACT_SPLIT_MAX_ABS_TOL, EXACT_SPLIT_REL_L2_TOL, dev, error_metrics, to_dev

pytestmark = pytest.mark.gpu

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
# |gpu - cpu| / rms(cpu) and relative L2 of the pre-activations: fp32 sums in another
# order, and elements far below their block's largest lose bits beyond the two-term
# split (measured: gate_up 5e-5 and 3.8e-6, partial, whose operands are heavier-tailed,
# 2.0e-4 and 2.3e-5)
PREACT_MAX_TOL = 6e-4
PREACT_L2_TOL = 6e-5


def _fns(lib):
    lib.vk_hip_moe_gateup_preact.restype = _I
    lib.vk_hip_moe_gateup_preact.argtypes = [_P] * 6 + [_I] * 8 + [_P]
    lib.vk_hip_moe_act_epilogue.restype = _I
    lib.vk_hip_moe_act_epilogue.argtypes = [_P] * 5 + [_I] * 4 + [_F, _I, _F, _F, _I, _P]
    lib.vk_hip_moe_down_preact.restype = _I
    lib.vk_hip_moe_down_preact.argtypes = [_P] * 6 + [_I] * 8 + [_P]
    lib.vk_hip_moe_combine.restype = _I
    lib.vk_hip_moe_combine.argtypes = [_P] * 6 + [_I] * 5 + [_P, ctypes.c_size_t, _P]
    return lib


def _case(cfg, T, seed, bs):
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed)
    A, lg = cfgs._inputs(cfg, T, seed)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    sids16, eids16, em16 = oracle.moe_align_block_size(ids, 16, cfg.E)
    sids, eids, em = oracle.moe_align_block_size(ids, bs, cfg.E)
    return w, A, ids, tw, (sids16[:em16], eids16[:em16 // 16], em16), (sids[:em].copy(), eids[:em // bs].copy(), em)


def _rows_map(sids16, sids, n_flat):
    """Sorted row (alignment of 16) of every flat index, and the same for the other block size."""
    p16 = np.full(n_flat, -1)
    p = np.full(n_flat, -1)
    r16 = np.nonzero(sids16 < n_flat)[0]
    p16[sids16[r16]] = r16
    r = np.nonzero(sids < n_flat)[0]
    p[sids[r]] = r
    return p16, p


def _rms_metrics(g, c):
    rms = float(np.sqrt(np.mean(c.astype(np.float64) ** 2)))
    d = g.astype(np.float64) - c.astype(np.float64)
    return float(np.abs(d).max() / rms), float(np.linalg.norm(d) / np.linalg.norm(c.astype(np.float64)))


@pytest.mark.parametrize("name,T,bs", [("c1", 1, 16), ("c1", 16, 16), ("c1", 64, 16), ("c4", 33, 16), ("c1", 300, 64),
                                       ("c0", 16, 16)])
def test_each_stage_against_the_oracle(hip_lib, name, T, bs):
    lib = _fns(hip_lib)
    cfg = synth.CONFIGS[name]
    H, I, k = cfg.H, cfg.I, cfg.top_k
    w, A, ids, tw, (s16, e16, em16), (sids, eids, em) = _case(cfg, T, 7100 + T, bs)
    wn = w.numpy()
    n_flat = T * k
    p16, p = _rows_map(s16, sids, n_flat)
    rng = np.random.default_rng(T)
    b13 = (rng.standard_normal((cfg.E, 2 * I)) * 0.5).astype(np.float32)
    b2 = (rng.standard_normal((cfg.E, H)) * 0.5).astype(np.float32)
    d = dict(A=to_dev(A), w13=to_dev(wn[0]), w13s=to_dev(wn[1]), w2=to_dev(wn[2]), w2s=to_dev(wn[3]),
             sids=to_dev(sids), eids=to_dev(eids), b13=to_dev(b13), b2=to_dev(b2))

    # stage 0a on the full K
    gu = torch.full((em, 2 * I), 7.0, dtype=torch.float32, device=dev())
    assert lib.vk_hip_moe_gateup_preact(d["A"].data_ptr(), d["w13"].data_ptr(), d["w13s"].data_ptr(),
                                        d["sids"].data_ptr(), d["eids"].data_ptr(), gu.data_ptr(), T, H, I, k,
                                        em, 0, H, bs, None) == 0, ve.last_error(lib)
    torch.cuda.synchronize()
    c_gu = oracle.moe_gateup(A, wn[0], wn[1], s16, e16, T, H, 0, H, I, k, em16)
    g_gu = gu.cpu().numpy()
    m, l2 = _rms_metrics(g_gu[p], c_gu[p16])
    print(f"{name} T={T} bs={bs}: gate_up max/rms {m:.2e} rel_l2 {l2:.2e}", end="; ")
    assert m <= PREACT_MAX_TOL and l2 <= PREACT_L2_TOL
    pad = np.setdiff1d(np.arange(em), p)
    assert np.all(g_gu[pad] == 7.0)                         # rows that are not routed are left alone

    # stage 0b on the oracle's own pre-activations (moved to this alignment's rows)
    for kw in (dict(), dict(swiglu_limit=7.0), dict(activation=1, beta=4.0, linear_beta=25.0)):
        src = np.zeros((em, 2 * I), np.float32)
        src[p] = c_gu[p16]
        act = torch.full((em, I), 0x1234, dtype=torch.int16, device=dev())
        d_src = to_dev(src)
        assert lib.vk_hip_moe_act_epilogue(d_src.data_ptr(), d["b13"].data_ptr(), act.data_ptr(),
                                           d["sids"].data_ptr(), d["eids"].data_ptr(), T, k, em, I,
                                           kw.get("swiglu_limit", 0.0), kw.get("activation", 0),
                                           kw.get("beta", 4.0), kw.get("linear_beta", 25.0), bs, None) == 0
        torch.cuda.synchronize()
        c_act = oracle.moe_act_epilogue(c_gu, b13, s16, e16, T, k, em16, I, **kw)
        g_act = act.cpu().numpy().view(np.uint16)
        ga, ca = g_act[p].astype(np.int32), c_act[p16].astype(np.int32)
        assert np.abs(ga - ca).max() <= 1, kw                  # one unit in the last place of bf16
        assert float(np.mean(ga != ca)) <= 0.02, kw
        assert np.all(g_act[pad] == 0x1234)

    # stage 1a on the oracle's act, full K
    c_act = oracle.moe_act_epilogue(c_gu, None, s16, e16, T, k, em16, I)
    act_rows = np.zeros((em, I), np.uint16)
    act_rows[p] = c_act[p16]
    part = torch.full((em, H), -3.0, dtype=torch.float32, device=dev())
    d_act = to_dev(act_rows)
    assert lib.vk_hip_moe_down_preact(d_act.data_ptr(), d["w2"].data_ptr(), d["w2s"].data_ptr(),
                                      d["sids"].data_ptr(), d["eids"].data_ptr(), part.data_ptr(), T, I, H, k,
                                      em, 0, I, bs, None) == 0, ve.last_error(lib)
    torch.cuda.synchronize()
    c_part = oracle.moe_down(c_act, wn[2], wn[3], s16, e16, T, I, 0, I, H, k, em16)
    g_part = part.cpu().numpy()
    m, l2 = _rms_metrics(g_part[p], c_part[p16])
    print(f"partial max/rms {m:.2e} rel_l2 {l2:.2e}")
    assert m <= PREACT_MAX_TOL and l2 <= PREACT_L2_TOL
    assert np.all(g_part[pad] == -3.0)

    # stage 1b on the oracle's partial rows: the reference's sum bit for bit
    tws16 = oracle.gather_sorted_weights(tw, s16)
    tws = oracle.gather_sorted_weights(tw, sids)
    src = np.zeros((em, H), np.float32)
    src[p] = c_part[p16]
    base = rng.standard_normal((T, H)).astype(np.float32)
    for bias, d_bias in ((None, None), (b2, d["b2"])):
        out = to_dev(base.copy())
        ws = torch.zeros(n_flat, dtype=torch.int32, device=dev())
        d_src, d_tws = to_dev(src), to_dev(tws)
        assert lib.vk_hip_moe_combine(d_src.data_ptr(), None if d_bias is None else d_bias.data_ptr(),
                                      d_tws.data_ptr(), d["sids"].data_ptr(), d["eids"].data_ptr(),
                                      out.data_ptr(), T, H, k, em, bs, ws.data_ptr(), ws.numel() * 4, None) == 0
        torch.cuda.synchronize()
        c_out = oracle.moe_combine(c_part, bias, tws16, s16, e16, T, H, k, em16, out=base.copy())
        assert np.array_equal(out.cpu().numpy().view(np.uint32), c_out.view(np.uint32)), bias is None


@pytest.mark.parametrize("name,T,bs,tp", [("c1", 1, 16, 2), ("c1", 32, 16, 2), ("c4", 7, 16, 2), ("c1", 200, 64, 3),
                                          ("c0", 16, 16, 2)])
def test_tensor_parallel_composition(hip_lib, name, T, bs, tp):
    """Every rank's K slice through the GEMM stages, the slices summed where the caller's
    all-reduce goes, the epilogues once: the fused oracle's layer."""
    lib = _fns(hip_lib)
    cfg = synth.CONFIGS[name]
    H, I, k = cfg.H, cfg.I, cfg.top_k
    w, A, ids, tw, (s16, e16, em16), (sids, eids, em) = _case(cfg, T, 7300 + T, bs)
    wn = w.numpy()
    n_flat = T * k
    rng = np.random.default_rng(T + 1)
    b13 = (rng.standard_normal((cfg.E, 2 * I)) * 0.5).astype(np.float32)
    b2 = (rng.standard_normal((cfg.E, H)) * 0.5).astype(np.float32)

    def slices(width):   # tp slices, each a multiple of 64 wide
        units = width // 64
        cuts = [64 * (units * r // tp) for r in range(tp + 1)]
        return [(cuts[r], cuts[r + 1] - cuts[r]) for r in range(tp) if cuts[r + 1] > cuts[r]]

    d_A, d_sids, d_eids = to_dev(A), to_dev(sids), to_dev(eids)
    d_b13, d_b2 = to_dev(b13), to_dev(b2)
    gu = torch.zeros((em, 2 * I), dtype=torch.float32, device=dev())
    for k_base, k_dim in slices(H):
        shard = np.ascontiguousarray(wn[0][:, :, k_base // 2:(k_base + k_dim) // 2])
        shard_s = np.ascontiguousarray(wn[1][:, :, k_base // 32:(k_base + k_dim) // 32])
        d_w, d_s = to_dev(shard), to_dev(shard_s)
        part = torch.zeros_like(gu)
        assert lib.vk_hip_moe_gateup_preact(d_A.data_ptr(), d_w.data_ptr(), d_s.data_ptr(), d_sids.data_ptr(),
                                            d_eids.data_ptr(), part.data_ptr(), T, H, I, k, em, k_base, k_dim,
                                            bs, None) == 0, ve.last_error(lib)
        gu += part                                            # the caller's all-reduce
        torch.cuda.synchronize()
    act = torch.zeros((em, I), dtype=torch.int16, device=dev())
    assert lib.vk_hip_moe_act_epilogue(gu.data_ptr(), d_b13.data_ptr(), act.data_ptr(), d_sids.data_ptr(),
                                       d_eids.data_ptr(), T, k, em, I, 0.0, 0, 4.0, 25.0, bs, None) == 0
    partial = torch.zeros((em, H), dtype=torch.float32, device=dev())
    for k_base, k_dim in slices(I):
        shard = np.ascontiguousarray(wn[2][:, :, k_base // 2:(k_base + k_dim) // 2])
        shard_s = np.ascontiguousarray(wn[3][:, :, k_base // 32:(k_base + k_dim) // 32])
        d_w, d_s = to_dev(shard), to_dev(shard_s)
        part = torch.zeros_like(partial)
        assert lib.vk_hip_moe_down_preact(act.data_ptr(), d_w.data_ptr(), d_s.data_ptr(), d_sids.data_ptr(),
                                          d_eids.data_ptr(), part.data_ptr(), T, I, H, k, em, k_base, k_dim,
                                          bs, None) == 0, ve.last_error(lib)
        partial += part
        torch.cuda.synchronize()
    out = torch.zeros((T, H), dtype=torch.float32, device=dev())
    ws = torch.zeros(n_flat, dtype=torch.int32, device=dev())
    d_tws = to_dev(oracle.gather_sorted_weights(tw, sids))
    assert lib.vk_hip_moe_combine(partial.data_ptr(), d_b2.data_ptr(), d_tws.data_ptr(), d_sids.data_ptr(),
                                  d_eids.data_ptr(), out.data_ptr(), T, H, k, em, bs, ws.data_ptr(),
                                  ws.numel() * 4, None) == 0
    torch.cuda.synchronize()
    tws16 = oracle.gather_sorted_weights(tw, s16)
    c_out, _ = oracle.fused_moe_mxfp4(A, *wn, s16, tws16, e16, T, H, I, k, em16, b13=b13, b2=b2)
    max_rel, rel_l2, nf = error_metrics(out.cpu().numpy(), c_out)
    print(f"{name} T={T} tp={tp}: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL


# ---- the same GEMM stages on prepacked weights (prefill-sized calls) -------------------------

def _prepacked_fns(lib):
    _fns(lib)
    lib.vk_hip_moe_preact_workspace_bytes.restype = ctypes.c_size_t
    lib.vk_hip_moe_preact_workspace_bytes.argtypes = [_I] * 4
    for name in ("vk_hip_moe_gateup_preact_prepacked", "vk_hip_moe_down_preact_prepacked"):
        fn = getattr(lib, name)
        fn.restype = _I
        fn.argtypes = [_P] * 4 + [_I] + [_P] * 3 + [_I] * 8 + [_P, ctypes.c_size_t, ctypes.c_uint, _P]
    return lib


def _prepack(lib, w, ws, stage):
    size_fn, pack_fn, _ = ve.resolve_prepack_fns(lib)
    E, rows, kb = w.shape
    n = int(size_fn(E, rows, kb * 2, stage))
    buf = torch.empty(n, dtype=torch.uint8, device=dev())
    assert pack_fn(w.data_ptr(), ws.data_ptr(), E, rows, kb * 2, stage, buf.data_ptr(), n, None) == 0
    return buf


# three FP6 terms represent a bf16 activation to 2^-13 of its block's largest: the sums then
# differ from the oracle's like the exact-split paths'; two terms (the second stage's
# default) leave 2^-10 of the block's largest per element
PREPACKED3_MAX_TOL, PREPACKED3_L2_TOL = 2e-3, 2e-4
PREPACKED2_MAX_TOL, PREPACKED2_L2_TOL = 2e-2, 2e-3


@pytest.mark.parametrize("name,T,bs,tp,raw", [("c1", 300, 128, 1, True), ("c1", 600, 128, 2, True),
                                              ("c4", 255, 64, 3, True), ("c1", 600, 128, 2, False),
                                              ("c4", 255, 64, 3, False), ("c1", 48, 16, 2, False),
                                              ("c1", 48, 32, 2, False), ("c4", 100, 32, 2, False)])
def test_prepacked_stages_against_the_oracle_and_in_composition(hip_lib, name, T, bs, tp, raw):
    """vk_hip_moe_gateup_preact_prepacked / _down_preact_prepacked: every rank's K slice of the
    weights prepacked as its own shard, the A / act slice addressed inside the full rows; each
    stage against the oracle's function of the same name on the same slice (rows that are not
    routed left as they were), and the composition (slices summed, epilogues once) against
    the fused oracle.  raw = False: the shard's raw tensors are not passed (one copy of the
    weights; decode-sized calls then run the decode kernels on the prepacked shard: in blocks
    of 32 the chunked kernel, whose linear part goes through the same two epilogues)."""
    lib = _prepacked_fns(hip_lib)
    cfg = synth.CONFIGS[name]
    H, I, k = cfg.H, cfg.I, cfg.top_k
    w, A, ids, tw, (s16, e16, em16), (sids, eids, em) = _case(cfg, T, 7500 + T, bs)
    wn = w.numpy()
    n_flat = T * k
    p16, p = _rows_map(s16, sids, n_flat)
    pad = np.setdiff1d(np.arange(em), p)
    rng = np.random.default_rng(T + 2)
    b13 = (rng.standard_normal((cfg.E, 2 * I)) * 0.5).astype(np.float32)
    b2 = (rng.standard_normal((cfg.E, H)) * 0.5).astype(np.float32)

    def slices(width):
        units = width // 64
        cuts = [64 * (units * r // tp) for r in range(tp + 1)]
        return [(cuts[r], cuts[r + 1] - cuts[r]) for r in range(tp) if cuts[r + 1] > cuts[r]]

    d_A, d_sids, d_eids = to_dev(A), to_dev(sids), to_dev(eids)
    gu = torch.zeros((em, 2 * I), dtype=torch.float32, device=dev())
    for k_base, k_dim in slices(H):
        d_w = to_dev(np.ascontiguousarray(wn[0][:, :, k_base // 2:(k_base + k_dim) // 2]))
        d_s = to_dev(np.ascontiguousarray(wn[1][:, :, k_base // 32:(k_base + k_dim) // 32]))
        packed = _prepack(lib, d_w, d_s, 0)
        need = int(lib.vk_hip_moe_preact_workspace_bytes(0, T, em, k_dim))
        ws = torch.empty(need, dtype=torch.uint8, device=dev())
        part = torch.full((em, 2 * I), 7.0, dtype=torch.float32, device=dev())
        assert lib.vk_hip_moe_gateup_preact_prepacked(
            d_A.data_ptr(), d_w.data_ptr() if raw else None, d_s.data_ptr() if raw else None, packed.data_ptr(),
            cfg.E, d_sids.data_ptr(),
            d_eids.data_ptr(), part.data_ptr(), T, H, I, k, em, k_base, k_dim, bs, ws.data_ptr(), need, 0,
            None) == 0, ve.last_error(lib)
        torch.cuda.synchronize()
        c_part = oracle.moe_gateup(A, wn[0][:, :, k_base // 2:(k_base + k_dim) // 2],
                                   wn[1][:, :, k_base // 32:(k_base + k_dim) // 32], s16, e16, T, H, k_base, k_dim,
                                   I, k, em16)
        g_part = part.cpu().numpy()
        m, l2 = _rms_metrics(g_part[p], c_part[p16])
        print(f"{name} T={T} slice {k_base}+{k_dim}: gate_up max/rms {m:.2e} rel_l2 {l2:.2e}")
        assert m <= PREPACKED3_MAX_TOL and l2 <= PREPACKED3_L2_TOL
        assert np.all(g_part[pad] == 7.0)                      # rows that are not routed are left alone
        part[to_dev(pad.astype(np.int64))] = 0.0
        gu += part                                              # the caller's all-reduce
    d_b13, d_b2 = to_dev(b13), to_dev(b2)
    act = torch.zeros((em, I), dtype=torch.int16, device=dev())
    assert lib.vk_hip_moe_act_epilogue(gu.data_ptr(), d_b13.data_ptr(), act.data_ptr(), d_sids.data_ptr(),
                                       d_eids.data_ptr(), T, k, em, I, 0.0, 0, 4.0, 25.0, bs, None) == 0
    torch.cuda.synchronize()
    act_np = act.cpu().numpy().view(np.uint16)
    act16 = np.zeros((em16, I), np.uint16)
    act16[p16] = act_np[p]
    partial = torch.zeros((em, H), dtype=torch.float32, device=dev())
    for k_base, k_dim in slices(I):
        d_w = to_dev(np.ascontiguousarray(wn[2][:, :, k_base // 2:(k_base + k_dim) // 2]))
        d_s = to_dev(np.ascontiguousarray(wn[3][:, :, k_base // 32:(k_base + k_dim) // 32]))
        packed = _prepack(lib, d_w, d_s, 1)
        need = int(lib.vk_hip_moe_preact_workspace_bytes(1, T, em, k_dim))
        ws = torch.empty(need, dtype=torch.uint8, device=dev())
        for flags, (mtol, ltol) in ((ve.MOE_SPLIT3, (PREPACKED3_MAX_TOL, PREPACKED3_L2_TOL)),
                                    (0, (PREPACKED2_MAX_TOL, PREPACKED2_L2_TOL))):
            part = torch.full((em, H), -3.0, dtype=torch.float32, device=dev())
            assert lib.vk_hip_moe_down_preact_prepacked(
                act.data_ptr(), d_w.data_ptr() if raw else None, d_s.data_ptr() if raw else None, packed.data_ptr(),
                cfg.E, d_sids.data_ptr(),
                d_eids.data_ptr(), part.data_ptr(), T, I, H, k, em, k_base, k_dim, bs, ws.data_ptr(), need, flags,
                None) == 0, ve.last_error(lib)
            torch.cuda.synchronize()
            c_part = oracle.moe_down(act16, wn[2][:, :, k_base // 2:(k_base + k_dim) // 2],
                                     wn[3][:, :, k_base // 32:(k_base + k_dim) // 32], s16, e16, T, I, k_base, k_dim,
                                     H, k, em16)
            g_part = part.cpu().numpy()
            m, l2 = _rms_metrics(g_part[p], c_part[p16])
            print(f"{name} T={T} slice {k_base}+{k_dim} flags {flags}: partial max/rms {m:.2e} rel_l2 {l2:.2e}")
            assert m <= mtol and l2 <= ltol
            assert np.all(g_part[pad] == -3.0)
        part[to_dev(pad.astype(np.int64))] = 0.0
        partial += part                                         # (the default arithmetic's)
    out = torch.zeros((T, H), dtype=torch.float32, device=dev())
    wsi = torch.zeros(n_flat, dtype=torch.int32, device=dev())
    d_tws = to_dev(oracle.gather_sorted_weights(tw, sids))
    assert lib.vk_hip_moe_combine(partial.data_ptr(), d_b2.data_ptr(), d_tws.data_ptr(), d_sids.data_ptr(),
                                  d_eids.data_ptr(), out.data_ptr(), T, H, k, em, bs, wsi.data_ptr(),
                                  wsi.numel() * 4, None) == 0
    torch.cuda.synchronize()
    tws16 = oracle.gather_sorted_weights(tw, s16)
    c_out, _ = oracle.fused_moe_mxfp4(A, *wn, s16, tws16, e16, T, H, I, k, em16, b13=b13, b2=b2)
    max_rel, rel_l2, nf = error_metrics(out.cpu().numpy(), c_out)
    print(f"{name} T={T} tp={tp} on prepacked shards: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= 8e-3 and rel_l2 <= 1e-3     # the bounds of the layer's default arithmetic
