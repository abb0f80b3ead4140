"""GPU parity of vk_hip_moe_route_layer_mxfp4 (router, alignment and the layer behind one
call) through the C ABI.  For a handful of tokens the first stage's kernel routes and aligns
for itself; up to 256 routed rows the router has its launch and the first stage's kernel
aligns from its ids.  The tables left (topk_ids, topk_w, sorted_ids, expert_ids, EM) must be
the oracle's bit for bit, every entry up to max_EM, exactly as the separate calls leave them,
and the layer's output inside the same bounds as theirs.  Shapes either side of every limit
of these forms (16 tokens, 256 routed rows, 256 experts, K = 3072 / 4096, a block size other
than 16), which run the separate kernels behind the same entry point; on the raw tensors and
on the prepacked form."""
from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

import test_gpu_configs as cfgs
from gpu_util import EXACT_SPLIT_MAX_ABS_TOL, EXACT_SPLIT_REL_L2_TOL, cpu_layer, dev, error_metrics, to_dev

pytestmark = pytest.mark.gpu


def _check(cfg, T, w, seed, block_size=None, expert_map=None, local_n=None, **kw):
    A_bits, lg = cfgs._inputs(cfg, T, seed)
    weights = (w.w13, w.w13_scale, w.w2, w.w2_scale)
    if expert_map is not None:
        own = to_dev(np.nonzero(expert_map >= 0)[0].astype(np.int64))
        weights = tuple(t[own].contiguous() for t in weights)
    fe = ve.FusedExperts(*weights, scratch=ve.CaptureSafeScratch(),
                         expert_map=None if expert_map is None else to_dev(expert_map),
                         local_num_experts=local_n, **kw)
    A = to_dev(A_bits, torch.bfloat16)
    out = torch.full((T, cfg.H), float("nan"), dtype=torch.float32, device=dev())
    got = fe.route_layer(A, to_dev(lg), cfg.top_k, block_size=block_size, out_fp32=out)
    torch.cuda.synchronize()
    _, ids, tw, sids, eids, out_em, max_em = got
    bs = block_size or fe.block_size_for(T, cfg.top_k)   # (with the prepacked weights: 32 beyond 256 routed rows)
    rid, rtw = oracle.route_topk(lg, cfg.top_k, True)
    assert np.array_equal(ids.cpu().numpy(), rid), "top-k indices differ from the oracle"
    assert np.array_equal(tw.cpu().numpy().view(np.uint32), rtw.view(np.uint32)), "router weights differ"
    s_ref, e_ref, em_ref = oracle.moe_align_block_size_with_map(rid.ravel(), cfg.E, bs, expert_map, max_EM=max_em)
    assert int(out_em.item()) == em_ref
    assert np.array_equal(sids.cpu().numpy(), s_ref), "sorted_ids differ (every entry up to max_EM is compared)"
    assert np.array_equal(eids.cpu().numpy(), e_ref), "expert_ids differ"
    tw_local = rtw if expert_map is None else np.where(expert_map[rid] >= 0, rtw, np.float32(0)).astype(np.float32)
    c = cpu_layer(A_bits, w.numpy(), rid, tw_local, threads=16)
    max_rel, rel_l2, nf = error_metrics(out.cpu().numpy(), c["out"])
    print(f"{cfg.name} T={T} bs={bs}: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL


@pytest.mark.parametrize("T", [1, 2, 3, 8, 16, 17, 64])
def test_route_layer_config1(T):
    cfg = synth.CONFIGS["c1"]
    _check(cfg, T, cfgs._weights(cfg, 1500), 6100 + T)


@pytest.mark.parametrize("name,T", [("c1", 17), ("c1", 33), ("c1", 64), ("c1", 65), ("c2", 64), ("c4", 33),
                                    ("c4", 42), ("c4", 43), ("c0", 128)])
@pytest.mark.parametrize("packed", [False, True])
def test_route_layer_aligning_in_the_first_stage(name, T, packed):
    """More than 16 tokens, up to 256 routed rows (c1 T=64, c4 T=42, c0 T=128 are the last that
    fit; c1 T=65 and c4 T=43 the first that do not): the router's launch, then the first stage
    aligning for itself."""
    cfg = synth.CONFIGS[name]
    kw = dict(prepack=True, keep_raw=False) if packed else {}
    _check(cfg, T, cfgs._weights(cfg), 6150 + T, **kw)


@pytest.mark.parametrize("T", [1, 7, 16, 33])
def test_route_layer_config2_zipf(T):
    cfg = synth.CONFIGS["c2"]       # 128 experts, a few of them popular
    _check(cfg, T, cfgs._weights(cfg), 6200 + T)


@pytest.mark.parametrize("T", [1, 16])
def test_route_layer_tiny_and_wide(T):
    cfg = synth.CONFIGS["c0"]       # 8 experts, top-2, K = 256
    _check(cfg, T, cfgs._weights(cfg, 1400), 6300 + T)
    cfg = synth.CONFIGS["c4"]       # K = 4096: its launch shape has no routed form
    _check(cfg, T, cfgs._weights(cfg, 4100), 6400 + T)


def test_route_layer_other_block_sizes_and_ties():
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    _check(cfg, 8, w, 6500, block_size=64)            # not the routed form's block size
    # every logit equal: ties go to the lowest expert, all tokens to the same four experts
    T = 16
    A_bits, _ = cfgs._inputs(cfg, T, 6501)
    lg = np.zeros((T, cfg.E), dtype=np.float32)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
    out, ids, tw, sids, eids, out_em, max_em = fe.route_layer(to_dev(A_bits, torch.bfloat16), to_dev(lg), cfg.top_k)
    torch.cuda.synchronize()
    rid, rtw = oracle.route_topk(lg, cfg.top_k, True)
    assert np.array_equal(ids.cpu().numpy(), rid) and (rid == np.arange(cfg.top_k)).all()
    s_ref, e_ref, em_ref = oracle.moe_align_block_size_with_map(rid.ravel(), cfg.E, 16, None, max_EM=max_em)
    assert int(out_em.item()) == em_ref == 64
    assert np.array_equal(sids.cpu().numpy(), s_ref) and np.array_equal(eids.cpu().numpy(), e_ref)
    c = cpu_layer(A_bits, w.numpy(), rid, rtw, threads=16)
    max_rel, rel_l2, nf = error_metrics(out.cpu().numpy(), c["out"])
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL


def test_route_layer_with_an_expert_map():
    cfg = synth.CONFIGS["c1"]
    rng = np.random.default_rng(66)
    local_n = cfg.E // 2
    emap = np.full(cfg.E, -1, dtype=np.int32)
    emap[np.sort(rng.permutation(cfg.E)[:local_n])] = np.arange(local_n, dtype=np.int32)
    for T in (1, 9, 40, 64):
        _check(cfg, T, cfgs._weights(cfg, 1500), 6600 + T, expert_map=emap, local_n=local_n)
    _check(cfg, 50, cfgs._weights(cfg, 1500), 6650, expert_map=emap, local_n=local_n, prepack=True, keep_raw=False)


def test_route_layer_equals_the_separate_calls():
    """The same inputs through route_align + the layer: identical tables, and an `out` that
    differs by the spread of the second stage's atomic adds only."""
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    for T in (1, 4, 16, 48):
        A_bits, lg = cfgs._inputs(cfg, T, 6700 + T)
        fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
        A, d_lg = to_dev(A_bits, torch.bfloat16), to_dev(lg)
        one = [t.clone() if isinstance(t, torch.Tensor) else t for t in fe.route_layer(A, d_lg, cfg.top_k)]
        ids, tw, sids, eids, out_em, max_em, bs = fe.route_align(d_lg, cfg.top_k, True)
        two = fe.apply(A, ids, tw, block_size=bs, aligned=(sids, eids, max_em))
        torch.cuda.synchronize()
        assert torch.equal(one[1], ids) and torch.equal(one[2].view(torch.int32), tw.view(torch.int32))
        assert torch.equal(one[3], sids) and torch.equal(one[4], eids) and torch.equal(one[5], out_em)
        a, b = one[0].double(), two.double()
        assert float((a - b).abs().max()) <= 1e-3 * float(b.pow(2).mean().sqrt())
