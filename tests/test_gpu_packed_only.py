"""Calls that pass the prepacked weights alone (the raw tensors null): one copy of the
weights.  The decode kernels' packed instantiations, the prepacked kernels and both exact
paths read the prepacked form; nothing may depend on the raw tensors.  Checked against the
oracle like the other calls, and against the same call with the raw tensors kept: the first
stage's output must be the same bits (the same products summed in the same order), the
layer's the same up to the order of the second stage's atomic additions at decode sizes and
the same bits at prefill sizes.  (The one-hot tests of test_gpu_prefill.py have paths on
the packed form alone as well: they pin the values, flagged units included.)"""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

import test_gpu_configs as cfgs
from gpu_util import (EXACT_SPLIT_MAX_ABS_TOL, EXACT_SPLIT_REL_L2_TOL, MAX_ABS_TOL, REL_L2_TOL, cpu_layer, dev,
                      error_metrics, to_dev)

pytestmark = pytest.mark.gpu

PACKED_ONLY = dict(prepack=True, keep_raw=False)


def _routed_rows(g, n_flat):
    return np.nonzero(g["sids"] < n_flat)[0]


@pytest.mark.parametrize("name,T", [("c0", 16), ("c1", 1), ("c1", 2), ("c1", 8), ("c1", 64), ("c2", 64),
                                    ("c4", 1), ("c4", 2), ("c4", 7), ("c4", 33)])
def test_decode_sizes_on_the_packed_form_alone(name, T):
    cfg = synth.CONFIGS[name]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6100 + T)
    g, wn = cfgs._check(cfg, T, w, A, lg, gpu_kw=PACKED_ONLY, tight=True)
    raw = cfgs._run_gpu(cfg, w, A, lg, None, None)
    rows = _routed_rows(g, T * cfg.top_k)
    same_shape = ve.moe_tile_query(0, cfg.H, cfg.I, T * cfg.top_k, packed=True)[0] == \
        ve.moe_tile_query(0, cfg.H, cfg.I, T * cfg.top_k)[0]
    if same_shape:   # the same products summed in the same order
        assert np.array_equal(g["act"][rows], raw["act"][rows]), "the first stage differs from the raw form's"
    else:            # (K shared between wavefronts in one form only: the sums are ordered differently)
        a = synth.bf16_bits_to_f32(g["act"][rows]).astype(np.float64)
        b = synth.bf16_bits_to_f32(raw["act"][rows]).astype(np.float64)
        assert np.linalg.norm(a - b) <= 2e-3 * np.linalg.norm(b)
    m, l2, nf = error_metrics(g["out"], raw["out"])
    assert nf and l2 <= 1e-5, (m, l2)


@pytest.mark.parametrize("name,T", [("c1", 300), ("c4", 255), ("c2", 512)])
def test_prefill_sizes_on_the_packed_form_alone(name, T):
    cfg = synth.CONFIGS[name]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6200 + T)
    a = cfgs._run_gpu(cfg, w, A, lg, None, True, **PACKED_ONLY)
    b = cfgs._run_gpu(cfg, w, A, lg, None, True, prepack=True)
    assert np.array_equal(a["out"].view(np.uint32), b["out"].view(np.uint32))
    assert np.all(np.isfinite(a["out"]))


@pytest.mark.parametrize("name,T", [("c4", 96), ("c2", 256), ("c2", 288), ("c4", 255)])
def test_few_rows_per_expert_beyond_512_rows(name, T):
    """A caller that gives the prepacked weights gets the decode kernels by rows per expert:
    with blocks of 16 (its own choice) up to 9 per expert (576 rows on 64 experts; 1024 and
    1152 on 128 with a few popular ones, where some experts have a dozen passes), with the
    policy's blocks of 32 up to 28 (1530 rows on 64 experts).  The exact-split bounds hold,
    and the call with blocks of 128 (the prepacked tile kernels) agrees."""
    cfg = synth.CONFIGS[name]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6300 + T)
    bs = ve.default_block_size(T, cfg.top_k, packed_experts=cfg.E, hidden=cfg.H, ispp=cfg.I)
    assert bs == 32 and T * cfg.top_k > 512
    t = cfgs._run_gpu(cfg, w, A, lg, 128, True, **PACKED_ONLY)
    for bs in ((16, 32) if T < 255 else (32,)):
        g, wn = cfgs._check(cfg, T, w, A, lg, gpu_kw=PACKED_ONLY, tight=True, block_size=bs, stagewise=(T == 255))
        m, l2, nf = error_metrics(g["out"], t["out"])
        assert nf and l2 <= 1.5e-3, (m, l2)


@pytest.mark.parametrize("T", [4, 300])
def test_values_outside_the_range_on_the_packed_form_alone(T):
    """inf/NaN codes and out-of-range scale bytes in some experts (flagged units, which keep
    the raw codes and scale bytes in the packed form) and rows with inf, NaN, huge and tiny
    values (their passes and segments take the exact path on units that are not flagged,
    whose codes and scale bytes are moved back): decode kernels (T = 4) and prepacked
    kernels (T = 300)."""
    cfg = synth.MoEConfig("t", 256, 512, 8, 2, (T,), "uniform")
    seed = 4300
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    r = synth.rand_u63(w.w13[0].numel(), seed, 32, dev()).reshape(w.w13[0].shape)
    w.w13[0][(r >> 10) % 4096 == 0] = 0x6E
    r = synth.rand_u63(w.w2[1].numel(), seed, 33, dev()).reshape(w.w2[1].shape)
    w.w2[1][(r >> 10) % 8192 == 0] = 0x7F
    w.w2_scale[2][::7, 1] = 200
    w.w13_scale[3][::5, 0] = 2
    A, lg = cfgs._inputs(cfg, T, seed)
    A = A.copy()
    A[0, 5] = 0x7F80
    A[1, 7] = 0x7FC0
    A[2, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[2, :]) * np.float32(2.0 ** 80))
    A[3, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[3, :]) * np.float32(2.0 ** -90))
    lg = lg.copy()
    lg[:, :4] += 4.0                      # the experts with flagged units take part at any T
    if T == 4:
        for t in range(T):
            lg[t, t % 4] += 20.0
            lg[t, (t + 1) % 4] += 19.0
    g = cfgs._run_gpu(cfg, w, A, lg, None, True, **PACKED_ONLY)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    for t in range(T):   # row by row: the rows differ by many orders of magnitude
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
    assert np.bincount(ids.ravel(), minlength=cfg.E)[:4].min() > 0


@pytest.mark.parametrize("T", [5, 300])
def test_a_wide_first_stage_on_the_packed_form_alone(T):
    """Rows of more than 4096 values do not fit the resident decode kernel's LDS: with the raw
    tensors such a call runs the tile kernels on them; without, the chunked decode kernel
    (T = 5) or the prepacked kernels (T = 300: 150 rows per expert), which need the workspace."""
    cfg = synth.MoEConfig("wide", 4608, 256, 4, 2, (T,), "uniform")
    seed = 6400
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    A, lg = cfgs._inputs(cfg, T, seed)
    g = cfgs._run_gpu(cfg, w, A, lg, None, True, **PACKED_ONLY)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    max_rel, rel_l2, nf = error_metrics(g["out"], c["out"])
    print(f"wide first stage, packed form alone, T={T}: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL
    if T == 5:
        return
    # and without a workspace the prefill-sized call is refused, not run on weights that are not there
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(), **PACKED_ONLY)
    d_ids, d_tw = to_dev(ids), to_dev(tw)
    sids, eids, _, max_em = fe.align(d_ids, 128)
    act = torch.zeros((max_em, cfg.I), dtype=torch.bfloat16, device=dev())
    out = torch.full((T, cfg.H), 3.0, dtype=torch.float32, device=dev())
    d_A = to_dev(A, torch.bfloat16)
    fe.lib.vk_set_last_error(0, b"")
    fe.moe_prepacked_fn(d_A.data_ptr(), None, None, None, None, d_ids.data_ptr(), d_tw.data_ptr(), act.data_ptr(),
                        out.data_ptr(), T, cfg.H, cfg.I, cfg.top_k, sids.data_ptr(), eids.data_ptr(), max_em,
                        0.0, 0, 4.0, 25.0, None, None, 128, None, 0, 0, fe.w13_packed.data_ptr(),
                        fe.w2_packed.data_ptr(), cfg.E, None)
    torch.cuda.synchronize()
    assert fe.lib.vk_last_error_code() == ve.VK_ERROR_INVALID_ARGUMENT
    assert bool((out == 3.0).all())


@pytest.mark.parametrize("name,T", [("c1", 1), ("c1", 8), ("c1", 16), ("c0", 16), ("c1", 40), ("c4", 1), ("c4", 2),
                                    ("c4", 16)])
def test_router_alignment_and_layer_in_one_call_on_the_packed_form_alone(name, T):
    cfg = synth.CONFIGS[name]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6500 + T)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(), **PACKED_ONLY)
    bs = ve.default_block_size(T, cfg.top_k)
    out, ids, tw, sids, eids, out_em, max_em = fe.route_layer(to_dev(A, torch.bfloat16), to_dev(lg), cfg.top_k,
                                                              block_size=bs)
    torch.cuda.synchronize()
    r_ids, r_tw = oracle.route_topk(lg, cfg.top_k, True)
    assert np.array_equal(ids.cpu().numpy(), r_ids)
    assert np.array_equal(tw.cpu().numpy().view(np.uint32), r_tw.view(np.uint32))
    s_ref, e_ref, em_ref = oracle.moe_align_block_size_with_map(r_ids.ravel(), cfg.E, bs, None, max_EM=max_em)
    assert int(out_em.item()) == em_ref
    assert np.array_equal(sids.cpu().numpy(), s_ref) and np.array_equal(eids.cpu().numpy(), e_ref)
    c = cpu_layer(A, w.numpy(), r_ids, r_tw, threads=16)
    max_rel, rel_l2, nf = error_metrics(out.cpu().numpy(), c["out"])
    print(f"{name} T={T}, one call, packed form alone: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL
