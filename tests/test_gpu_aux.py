"""GPU parity of the MXFP4 MoE orchestration ops (device counterparts of the reference's
moe_aux.cpp) and of the W4A4 mode of the layer, through the C ABI.

Bit-exact: quantised codes and scale bytes (token and sorted order), the routed combine.
W4A4 layer: against the oracle run on the same quantised activations
(`oracle.set_act_model(1)`), where only the order of the fp32 sums differs."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

import test_gpu_configs as cfgs
from gpu_util import MAX_ABS_TOL, REL_L2_TOL, cpu_layer, dev, edge_tokens, error_metrics, to_dev

pytestmark = pytest.mark.gpu

_P, _I = ctypes.c_void_p, ctypes.c_int


def _edge_rows(M, hidden, seed):
    """Activations with everything the quantiser has cases for."""
    A = synth.make_activations(M, hidden, seed)
    f = synth.bf16_bits_to_f32(A)
    rng = np.random.default_rng(seed)
    A[0, :32] = 0                                                     # a zero group
    A[1, 40] = 0x7F80                                                 # inf: its group is zero
    A[2, 9] = 0x7FC1                                                  # NaN inside a finite group
    A[3, :] = rng.integers(0, 128, hidden).astype(np.uint16)          # bf16 subnormals
    A[4, :] = synth.f32_to_bf16_bits(f[4] * np.float32(2.0 ** 100))
    A[5, :] = synth.f32_to_bf16_bits(f[5] * np.float32(2.0 ** -100))
    A[6, :32] = synth.f32_to_bf16_bits(np.array([3, .125, .625, 1.25, 1.75, 2.5, -.125, -.124, -0.0, 0.0] + [0.1] * 22, np.float32))
    A[7, :64] = synth.f32_to_bf16_bits(np.r_[np.full(32, 1.5), np.full(32, 1.5078125)].astype(np.float32))  # m = 1.5 and above
    A[8, 0] = 0x7F00                                                  # 2^127 next to small values
    A[9, :32] = 0x8000                                                # negative zeros
    A[10, 3] = 0xFF80                                                 # -inf
    A[11, :32] = rng.integers(0, 65536, 32).astype(np.uint16)         # arbitrary bit patterns
    A[12:16] = rng.integers(0, 65536, (4, hidden)).astype(np.uint16)
    return A


def test_quant_bitwise(hip_lib):
    fn = hip_lib.vk_hip_mxfp4_moe_quant
    fn.restype = _I
    fn.argtypes = [_P, _P, _P, _I, _I, _I, _P]
    M, hidden = 48, 2880
    A = _edge_rows(M, hidden, 301)
    packed = torch.zeros((M, hidden // 2), dtype=torch.uint8, device=dev())
    scales = torch.zeros((M, hidden // 32), dtype=torch.uint8, device=dev())
    d_A = to_dev(A)
    assert fn(d_A.data_ptr(), packed.data_ptr(), scales.data_ptr(), M, hidden, 32, None) == 0
    torch.cuda.synchronize()
    rp, rs = oracle.mxfp4_moe_quant(A)
    gs, gp = scales.cpu().numpy(), packed.cpu().numpy()
    assert np.array_equal(gs, rs), f"scale bytes differ at (row, group) {np.argwhere(gs != rs)[:10].tolist()}"
    assert np.array_equal(gp, rp), f"codes differ at (row, byte) {np.argwhere(gp != rp)[:10].tolist()}"
    assert fn(None, None, None, 4, 64, 16, None) == ve.VK_ERROR_UNSUPPORTED


def test_sorted_quant_and_scatter_reduce_bitwise(hip_lib):
    sq = hip_lib.vk_hip_mxfp4_moe_sorted_quant
    sq.restype = _I
    sq.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P]
    sr = hip_lib.vk_hip_mxfp4_moe_scatter_reduce
    sr.restype = _I
    sr.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _P, ctypes.c_size_t, _P]
    rng = np.random.default_rng(5)
    M, hidden, top_k, E = 70, 512, 4, 16
    A = _edge_rows(M, hidden, 302)
    ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
    sids, _, em = oracle.moe_align_block_size(ids, 16, E)
    sids = sids[:em].copy()
    sids[5] = -3                                    # a negative id is padding too
    packed = torch.full((em, hidden // 2), 7, dtype=torch.uint8, device=dev())
    scales = torch.full((em, hidden // 32), 7, dtype=torch.uint8, device=dev())
    d_A, d_sids = to_dev(A), to_dev(sids)      # (kept alive until the synchronisation)
    assert sq(d_A.data_ptr(), d_sids.data_ptr(), packed.data_ptr(), scales.data_ptr(), M, hidden,
              32, top_k, em, None) == 0
    torch.cuda.synchronize()
    rp, rs = oracle.mxfp4_moe_sorted_quant(A, sids, top_k)
    assert np.array_equal(packed.cpu().numpy(), rp) and np.array_equal(scales.cpu().numpy(), rs)

    width = 2880
    partial = (rng.standard_normal((em, width)) * 100).astype(np.float32)
    tws = rng.random(em).astype(np.float32)
    base = rng.standard_normal((M, width)).astype(np.float32)      # the call accumulates
    out = to_dev(base.copy())
    ws = torch.zeros(M * top_k, dtype=torch.int32, device=dev())
    d_partial, d_tws = to_dev(partial), to_dev(tws)
    assert sr(d_partial.data_ptr(), d_tws.data_ptr(), d_sids.data_ptr(), out.data_ptr(), M,
              width, top_k, em, ws.data_ptr(), ws.numel() * 4, None) == 0
    torch.cuda.synchronize()
    ref = oracle.mxfp4_moe_scatter_reduce(partial, tws, sids, M, top_k, out=base.copy())
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    assert sr(None, None, None, None, M, width, top_k, em, None, 0, None) == ve.VK_ERROR_INVALID_ARGUMENT


@pytest.mark.parametrize("hidden", [512, 2880, 76])
def test_sort_and_sort_scales_bitwise(hip_lib, hidden):
    """mxfp4_moe_sort / mxfp4_moe_sort_scales on the device: rows gathered into sorted
    order, padding rows (ids at or beyond M * top_k, negative ids) zeroed; byte for byte
    the oracle's.  hidden = 76: rows that are no multiple of 16 bytes (the byte-wise
    kernel), scale rows of 2 bytes."""
    st = hip_lib.vk_hip_mxfp4_moe_sort
    st.restype = _I
    st.argtypes = [_P, _P, _P, _I, _I, _I, _I, _P]
    ss = hip_lib.vk_hip_mxfp4_moe_sort_scales
    ss.restype = _I
    ss.argtypes = [_P, _P, _P, _I, _I, _I, _I, _P]
    rng = np.random.default_rng(hidden)
    M, top_k, E = 70, 4, 16
    A = rng.integers(0, 65536, (M, hidden)).astype(np.uint16)
    n_groups = max(hidden // 32, 1)
    scales = rng.integers(0, 256, (M, n_groups)).astype(np.uint8)
    ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
    sids, _, em = oracle.moe_align_block_size(ids, 16, E)
    sids = sids[:em].copy()
    sids[3] = -1
    d_A, d_s, d_sids = to_dev(A), to_dev(scales), to_dev(sids)
    a_sorted = torch.full((em, hidden), 0x1234, dtype=torch.int16, device=dev())
    s_sorted = torch.full((em, n_groups), 9, dtype=torch.uint8, device=dev())
    assert st(d_A.data_ptr(), d_sids.data_ptr(), a_sorted.data_ptr(), M, hidden, top_k, em, None) == 0
    assert ss(d_s.data_ptr(), d_sids.data_ptr(), s_sorted.data_ptr(), M, n_groups, top_k, em, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(a_sorted.cpu().numpy().view(np.uint16), oracle.mxfp4_moe_sort(A, sids, top_k))
    assert np.array_equal(s_sorted.cpu().numpy(), oracle.mxfp4_moe_sort_scales(scales, sids, top_k))
    assert st(None, None, None, M, hidden, 0, em, None) == ve.VK_ERROR_INVALID_ARGUMENT
    assert ss(None, None, None, M, n_groups, top_k, em, None) == ve.VK_ERROR_INVALID_ARGUMENT
    assert st(None, None, None, M, hidden, top_k, 0, None) == 0              # nothing to do


def test_scatter_reduce_q_bitwise(hip_lib):
    """mxfp4_moe_scatter_reduce_q on the device: the routed combine of a quantised partial,
    dequantised inline; the same bits as the oracle (each product and each sum rounded on
    its own, rows in ascending order), with every code (inf and NaN included), scale bytes
    0, 1, 254 and 0xFF, and an `out` that already holds values."""
    fn = hip_lib.vk_hip_mxfp4_moe_scatter_reduce_q
    fn.restype = _I
    fn.argtypes = [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, ctypes.c_size_t, _P]
    rng = np.random.default_rng(77)
    M, width, top_k, E = 70, 2880, 4, 16
    ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
    sids, _, em = oracle.moe_align_block_size(ids, 16, E)
    sids = sids[:em].copy()
    sids[7] = -2
    pq = rng.integers(0, 256, (em, width // 2)).astype(np.uint8)
    fin = np.array(synth.FINITE_CODES, dtype=np.uint8)
    finite_rows = np.arange(em) % 4 != 0                               # three rows in four: finite codes only
    pq[finite_rows] = fin[pq[finite_rows] % 12 & 15] | (fin[(pq[finite_rows] >> 4) % 12] << 4)
    ps = rng.integers(110, 140, (em, width // 32)).astype(np.uint8)
    ps[:, 0] = 0
    ps[:, 1] = 1
    ps[:, 2] = 254
    ps[:, 3] = 255
    tws = rng.random(em).astype(np.float32)
    base = rng.standard_normal((M, width)).astype(np.float32)
    out = to_dev(base.copy())
    ws = torch.zeros(M * top_k, dtype=torch.int32, device=dev())
    d_pq, d_ps, d_tws, d_sids = to_dev(pq), to_dev(ps), to_dev(tws), to_dev(sids)
    assert fn(d_pq.data_ptr(), d_ps.data_ptr(), d_tws.data_ptr(), d_sids.data_ptr(), out.data_ptr(), M, width,
              top_k, em, 32, ws.data_ptr(), ws.numel() * 4, None) == 0, ve.last_error(hip_lib)
    torch.cuda.synchronize()
    ref = oracle.mxfp4_moe_scatter_reduce_q(pq, ps, tws, sids, M, top_k, out=base.copy())
    got = out.cpu().numpy()
    nan_g, nan_r = np.isnan(got), np.isnan(ref)
    assert np.array_equal(nan_g, nan_r) and nan_r.any() and not nan_r.all()
    assert np.array_equal(got.view(np.uint32)[~nan_r], ref.view(np.uint32)[~nan_r])
    assert fn(None, None, None, None, None, M, width, top_k, em, 32, None, 0, None) == ve.VK_ERROR_INVALID_ARGUMENT
    assert fn(None, None, None, None, None, M, width, top_k, em, 16, None, 0, None) == ve.VK_ERROR_UNSUPPORTED


def _check_w4a4(cfg, T, w, A_bits, logits, sample=128, wn=None):
    g = cfgs._run_gpu(cfg, w, A_bits, logits, None, True, prepack=True, w4a4=True)
    ids, tw = oracle.route_topk(logits, cfg.top_k, True)
    assert np.array_equal(g["ids"], ids)
    rows = np.arange(T) if sample is None or sample >= T else edge_tokens(g, T * cfg.top_k, cfg.top_k, sample, T)
    wn = w.numpy() if wn is None else wn
    oracle.set_act_model(1)
    try:
        cm = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16)
    finally:
        oracle.set_act_model(0)
    m_rel, m_l2, nf = error_metrics(g["out"][rows], cm["out"])
    c = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16)
    b_rel, b_l2, _ = error_metrics(g["out"][rows], c["out"])
    print(f"{cfg.name} T={T} W4A4 rows checked {rows.size}: vs oracle on the quantised activations "
          f"max_abs/rms={m_rel:.3e} rel_l2={m_l2:.3e}; vs the bf16-activation oracle rel_l2={b_l2:.3e}")
    # same operands on both sides: what differs is the order of the sums, and bf16 roundings
    # of act that fall the other way (each then moves its quantised value by a code step)
    assert nf and m_rel <= MAX_ABS_TOL and m_l2 <= REL_L2_TOL
    return g, wn


@pytest.mark.parametrize("T", [200, 513])
def test_w4a4_layer_config1(T):
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, 6100 + T)
    _check_w4a4(cfg, T, w, A, lg)


def test_w4a4_layer_config3():
    cfg = synth.CONFIGS["c3"]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, 4096, 3000)
    _check_w4a4(cfg, 4096, w, A, lg, sample=96)


def test_w4a4_first_stage_matches_the_model_closely():
    """The first stage alone has no rounding between quantisation and output but the
    fp32 sums: act against the oracle's act on the quantised activations."""
    cfg = synth.CONFIGS["c1"]
    T = 200
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, 6200)
    g = cfgs._run_gpu(cfg, w, A, lg, 16, True, prepack=True, w4a4=True)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    oracle.set_act_model(1)
    try:
        c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    finally:
        oracle.set_act_model(0)
    real = c["sorted_ids"] < T * cfg.top_k
    ga = synth.bf16_bits_to_f32(g["act"][:c["EM"]][real]).astype(np.float64)
    ca = synth.bf16_bits_to_f32(c["act"][real]).astype(np.float64)
    rms = float(np.sqrt(np.mean(ca ** 2)))
    excess = np.abs(ga - ca) - (1e-3 * rms + 2.0 ** -7 * np.abs(ca))
    assert float(excess.max()) <= 0.0
    assert float(np.linalg.norm(ga - ca) / np.linalg.norm(ca)) <= 2e-3


def test_w4a4_rows_outside_the_range_take_the_exact_path():
    cfg = synth.MoEConfig("t", 256, 512, 8, 2, (300,), "uniform")
    T, seed = 300, 6300
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    r = synth.rand_u63(w.w13[0].numel(), seed, 32, dev()).reshape(w.w13[0].shape)
    w.w13[0][(r >> 10) % 4096 == 0] = 0x6E       # inf codes in one expert: flagged units
    A, lg = cfgs._inputs(cfg, T, seed)
    A = A.copy()
    A[2, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[2, :]) * np.float32(2.0 ** 80))    # scale byte > 190
    A[3, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[3, :]) * np.float32(2.0 ** -90))   # < 64
    A[4, :] = 0
    A[5, 7] = 0x7F80                              # an inf: its group quantises to zero
    g = cfgs._run_gpu(cfg, w, A, lg, None, True, prepack=True, w4a4=True)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    oracle.set_act_model(1)
    try:
        c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    finally:
        oracle.set_act_model(0)
    for t in range(T):
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
