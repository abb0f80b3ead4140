"""GPU parity of the fused MXFP4 MoE layer on the larger configurations.

Where the CPU oracle would need minutes (prefill sizes), the layer runs at
full size on the GPU and the oracle computes a seeded sample of the tokens:
a token's output row depends on that token's activations, its routing and
the weights only, so `oracle(A[sample], ids[sample], w[sample])` must equal
`gpu_out[sample]`.  The router and the alignment are always compared in full,
bit for bit.  Full-size runs are also checked through batch-size independence:
the inputs of a shorter batch are a prefix of the longer one's (the generator
is counter based), so the shared rows must agree.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

from gpu_util import (EXACT_SPLIT_MAX_ABS_TOL, EXACT_SPLIT_REL_L2_TOL, MAX_ABS_TOL, REL_L2_TOL, cpu_layer,
                      dev, edge_tokens, error_metrics, to_dev)

pytestmark = pytest.mark.gpu

_WEIGHTS = {}


def _weights(cfg, seed=None, **kw):
    """Device weights of a config (one seed for all its batch sizes), cached."""
    seed = int(cfg.name[1:]) * 1000 if seed is None else seed
    key = (cfg.name, seed, tuple(sorted(kw.items())))
    if key not in _WEIGHTS:
        _WEIGHTS.clear()  # one config's weights at a time: the largest set is 5.6 GB
        _WEIGHTS[key] = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev(), **kw)
    return _WEIGHTS[key]


def _run_gpu(cfg, w, A_bits, logits, block_size=None, use_workspace=None, **kw):
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(), **kw)
    if use_workspace is not None:
        fe.use_workspace = use_workspace
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(logits), cfg.top_k, True)
    T = A.shape[0]
    bs = ve.default_block_size(T, cfg.top_k) if block_size is None else block_size
    sids, eids, out_em, max_em = fe.align(ids, bs)
    out = fe.apply(A, ids, tw, block_size=bs)
    torch.cuda.synchronize()
    act = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16, device=dev())
    return dict(out=out.cpu().numpy(), ids=ids.cpu().numpy(), tw=tw.cpu().numpy(),
                sids=sids.cpu().numpy(), eids=eids.cpu().numpy(), EM=int(out_em.item()),
                max_EM=max_em, bs=bs,
                act=act.view(torch.int16).cpu().numpy().view(np.uint16).reshape(max_em, fe.ispp))


def _check_stagewise(cfg, T, g, A_bits, wn, tw):
    """Stage by stage, for inputs whose outputs are dominated by single terms (block scales
    of 2^+-20).  There one rounding of a bf16 act value the other way, which any change of
    the summation order can cause, moves an output by a percent, and sums cancel by factors
    of thousands, so the end-to-end figure says little.  Instead:
    (1) the first stage against exact arithmetic: with g, u the float64 dot products and
        Sg, Su the sums of the absolute values of their terms, every act value must be
        f(g, u) within the change of f under dg = eps * Sg, du = eps * Su (eps = 2^-13: the
        matrix cores align the four blocks of a K step and keep about 16 bits below the
        largest) plus two bf16 ulps;
    (2) the second stage against the oracle's second stage run on the GPU's own act."""
    n_flat = T * cfg.top_k
    eps = 2.0 ** -13
    Af = synth.bf16_bits_to_f32(A_bits).astype(np.float64)
    bs = g["bs"]
    worst = 0.0
    for blk, e in enumerate(g["eids"]):
        rows = np.arange(blk * bs, (blk + 1) * bs)
        rows = rows[g["sids"][rows] < n_flat]
        if e < 0 or rows.size == 0:
            continue
        wd = synth.bf16_bits_to_f32(oracle.dequant_weight_tile(wn[0][e], wn[1][e], 2 * cfg.I, cfg.H))
        wd = wd.astype(np.float64)                      # [K, 2I]
        a = Af[g["sids"][rows] // cfg.top_k]
        gu, s_gu = a @ wd, np.abs(a) @ np.abs(wd)
        gg, uu, dg, du = gu[:, :cfg.I], gu[:, cfg.I:], eps * s_gu[:, :cfg.I], eps * s_gu[:, cfg.I:]
        silu = gg / (1.0 + np.exp(-gg))
        ref = silu * uu
        tol = 1.1 * (np.abs(uu) + du) * dg + (np.abs(silu) + 1.1 * dg) * du + 2.0 ** -7 * np.abs(ref) + 1e-30
        got = synth.bf16_bits_to_f32(g["act"][rows]).astype(np.float64)
        worst = max(worst, float(np.max(np.abs(got - ref) / tol)))
    print(f"{cfg.name} T={T} first stage against float64: worst |error| / bound = {worst:.3f}")
    assert worst <= 1.0, "act is outside the rounding bound of the exact gate/up products"
    eids16 = np.repeat(g["eids"], g["bs"] // 16).astype(np.int32)
    EM = g["max_EM"]
    partial = oracle.moe_down(g["act"], wn[2], wn[3], g["sids"], eids16, T, cfg.I, 0, cfg.I, cfg.H,
                              cfg.top_k, EM)
    tws = oracle.gather_sorted_weights(tw, g["sids"])
    ref = oracle.moe_combine(partial, None, tws, g["sids"], eids16, T, cfg.H, cfg.top_k, EM)
    max_rel, rel_l2, nf = error_metrics(g["out"], ref)
    print(f"{cfg.name} T={T} second stage on the GPU's act: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL


def _check(cfg, T, w, A_bits, logits, sample=None, block_size=None, weights_np=None,
           gpu_kw=None, cpu_kw=None, seed=0, stagewise=False, use_workspace=None, tight=False):
    g = _run_gpu(cfg, w, A_bits, logits, block_size, use_workspace, **(gpu_kw or {}))
    # router and alignment: bit for bit, full size
    ids, tw = oracle.route_topk(logits, cfg.top_k, True)
    assert np.array_equal(g["ids"], ids), "top-k indices differ from the oracle"
    assert np.array_equal(g["tw"].view(np.uint32), tw.view(np.uint32)), "router weights differ"
    s_ref, e_ref, em_ref = oracle.moe_align_block_size_with_map(
        ids.ravel(), cfg.E, g["bs"], None, max_EM=g["max_EM"])
    assert g["EM"] == em_ref
    assert np.array_equal(g["sids"], s_ref) and np.array_equal(g["eids"], e_ref)
    # the layer: all tokens, or a seeded sample of them
    # (sampled rows include the places where a tile kernel breaks: window and tile edges,
    # the last rows of experts, the most and the least popular expert)
    rows = np.arange(T)
    if sample is not None and sample < T:
        rows = edge_tokens(g, T * cfg.top_k, cfg.top_k, sample, seed)
    wn = w.numpy() if weights_np is None else weights_np
    c = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16, **(cpu_kw or {}))
    max_rel, rel_l2, nf = error_metrics(g["out"][rows], c["out"])
    print(f"{cfg.name} T={T} bs={g['bs']} rows checked {rows.size}: "
          f"max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    if stagewise:
        assert rows.size == T and nf and rel_l2 <= REL_L2_TOL
        _check_stagewise(cfg, T, g, A_bits, wn, tw)
    else:
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL
        if tight:  # these paths split the activations exactly: only the order of the sums differs
            assert max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL
    return g, wn


def _inputs(cfg, T, seed):
    A = synth.make_activations(T, cfg.H, seed)
    lg = synth.make_logits(cfg.logits, T, cfg.E, seed, A, cfg.H)
    return A, lg


# ---- config 2: 128 experts, Zipf popularity -----------------------------------

def test_config2_zipf_all_sizes():
    cfg = synth.CONFIGS["c2"]
    w = _weights(cfg)
    wn = None
    prev = None
    for T, sample in ((4096, 128), (512, 128), (64, None)):
        A, lg = _inputs(cfg, T, 2000)
        g, wn = _check(cfg, T, w, A, lg, sample=sample, weights_np=wn, tight=True)
        counts = np.bincount(g["ids"].ravel(), minlength=cfg.E)
        if T == 4096:
            assert counts.max() > 8 * np.median(counts), "the Zipf routing should be imbalanced"
        if prev is not None:  # same first rows as the longer batch
            m, l2, nf = error_metrics(g["out"], prev[:T])
            assert nf and m <= MAX_ABS_TOL and l2 <= REL_L2_TOL
        prev = g["out"]


# ---- config 3: wide hidden, 256 small experts, prefill ------------------------

@pytest.mark.parametrize("T", [4096, 16384])
def test_config3_prefill(T):
    cfg = synth.CONFIGS["c3"]
    w = _weights(cfg)
    A, lg = _inputs(cfg, T, 3000)
    g, _ = _check(cfg, T, w, A, lg, sample=128, tight=True)
    assert np.all(np.isfinite(g["out"]))
    # weighted-combine sanity at full size: the routing weights of a token sum to 1,
    # so scaling them by 2 through a second call must double the output
    if T == 4096:
        fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
        ids = to_dev(g["ids"])
        out2 = fe.apply(to_dev(A, torch.bfloat16), ids, to_dev(2.0 * g["tw"])).cpu().numpy()
        m, l2, nf = error_metrics(out2, 2.0 * g["out"])
        assert nf and l2 <= 1e-5, (m, l2)


# ---- config 4: robustness sweep ------------------------------------------------

def _extreme_weights(cfg, seed):
    """Block scales with exponents +-20 and all-zero blocks sprinkled in."""
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    for t_codes, t_scale, stream in ((w.w13, w.w13_scale, 11), (w.w2, w.w2_scale, 12)):
        n = t_scale.numel()
        r = synth.rand_u63(n, seed, stream, dev()).reshape(t_scale.shape)
        sel = (r >> 20) % 100
        t_scale[sel == 0] = 107   # 2^-20
        t_scale[sel == 1] = 147   # 2^+20
        zero = (sel == 2)
        blocks = t_codes.reshape(*t_scale.shape, 16)
        blocks[zero] = 0          # all-zero block
    return w


@pytest.mark.parametrize("T", [1, 7, 33, 255, 1000, 8191])
def test_config4_ragged(T):
    cfg = synth.CONFIGS["c4"]
    seed = 4000
    key = ("c4x", seed)
    if key not in _WEIGHTS:
        _WEIGHTS.clear()
        _WEIGHTS[key] = _extreme_weights(cfg, seed)
    w = _WEIGHTS[key]
    A, lg = _inputs(cfg, T, seed)
    if T == 7:
        lg[:] = lg[0]                      # every token on the same six experts
    if T == 33:
        lg[:, cfg.E // 2:] = -30.0         # half of the experts receive nothing
    if T == 255:
        lg[:, 5] += 12.0                   # one expert in every token's top-k
    g, _ = _check(cfg, T, w, A, lg, sample=None if T <= 255 else 128, stagewise=T <= 255)
    counts = np.bincount(g["ids"].ravel(), minlength=cfg.E)
    if T == 7:
        assert np.count_nonzero(counts) == cfg.top_k
    if T == 33:
        assert counts[cfg.E // 2:].sum() == 0
    if T == 255:
        assert counts[5] == T


# ---- epilogue variants, block sizes ---------------------------------------------

@pytest.mark.parametrize("T", [8, 200])
@pytest.mark.parametrize("variant", ["bias", "limit", "situ", "situ_bias"])
def test_epilogue_variants(variant, T):
    """T = 8: the decode kernels; T = 200 (800 routed rows): the tile kernels of the
    workspace path, whose second stage adds its bias before the combine pass."""
    cfg = synth.CONFIGS["c1"]
    seed = 1500
    w = _weights(cfg, seed)
    A, lg = _inputs(cfg, T, seed)
    b13 = (synth.rand_normal((cfg.E, 2 * cfg.I), seed, 21) * 0.5).astype(np.float32)
    b2 = (synth.rand_normal((cfg.E, cfg.H), seed, 22) * 0.5).astype(np.float32)
    gpu_kw, cpu_kw = {}, {}
    if "bias" in variant:
        gpu_kw.update(b13=to_dev(b13), b2=to_dev(b2))
        cpu_kw.update(b13=b13, b2=b2)
    if variant == "limit":
        gpu_kw.update(swiglu_limit=1.5)
        cpu_kw.update(swiglu_limit=1.5)
    if "situ" in variant:
        gpu_kw.update(activation="situ", beta=3.0, linear_beta=20.0)
        cpu_kw.update(activation=1, beta=3.0, linear_beta=20.0)
    _check(cfg, T, w, A, lg, sample=32 if T > 32 else None, gpu_kw=gpu_kw, cpu_kw=cpu_kw)


@pytest.mark.parametrize("bs", [16, 32, 64, 128])
def test_block_sizes(bs):
    cfg = synth.CONFIGS["c1"]
    T, seed = 40, 1600
    w = _weights(cfg, 1500)
    A, lg = _inputs(cfg, T, seed)
    _check(cfg, T, w, A, lg, block_size=bs)


def test_decode_with_more_sorted_rows_than_the_kernel_copies_to_lds():
    """Many experts and a short K.  The decode kernel copies the head of sorted_ids to LDS
    (1024 ids per K step of its operand planes: 2048 here) and reads the ids of the runs
    behind that from memory; both ways are taken here, in both stages, and with more than
    64 blocks the run listing takes several rounds."""
    cfg = synth.MoEConfig("c9", 256, 256, 256, 8, (40,), "uniform")
    T, seed = 40, 9040
    w = _weights(cfg, 9000)
    A, lg = _inputs(cfg, T, seed)
    g, _ = _check(cfg, T, w, A, lg)
    assert g["bs"] == 16 and T * cfg.top_k <= 512, "not a decode-sized call"
    assert g["EM"] > 2048 + 64, "every run's ids fit the copy in LDS"


def test_decode_with_more_runs_than_workgroups():
    """512 experts, 480 routed rows: more than 256 blocks of 16 rows, each a run of its own,
    so the runs cannot have workgroups of their own and the (run, unit) space is cut
    evenly, a workgroup's slice spanning several runs."""
    cfg = synth.MoEConfig("c8", 256, 256, 512, 8, (60,), "uniform")
    T, seed = 60, 8060
    w = _weights(cfg, 8000)
    A, lg = _inputs(cfg, T, seed)
    g, _ = _check(cfg, T, w, A, lg)
    assert g["bs"] == 16 and T * cfg.top_k <= 512, "not a decode-sized call"
    assert g["EM"] // 16 > 256, "fewer runs than the device has compute units"


@pytest.mark.parametrize("T", [1, 2, 9, 40])
def test_decode_with_k_shared_between_wavefronts(T):
    """Every K-split shape of the decode kernel, put in the tuning store for the call's size:
    one token (a unit per 2 to 8 wavefronts, what the compiled-in rule chooses it for), and
    sizes where a workgroup has more units than half its wavefronts and takes them a few at
    a time.  Weight scales outside the fast range make some units leave the fast path in
    one part of K only."""
    cfg = synth.MoEConfig("c9", 1536, 1024, 8, 2, (T,), "uniform")
    w = _weights(cfg, 9001 if T == 9 else 9000)
    if T == 9 and not getattr(w, "tiny_scales_set", False):
        for t in (w.w13_scale, w.w2_scale):  # (tiny ones: nothing overflows)
            special = torch.tensor([0, 1, 63], dtype=torch.uint8, device=dev())
            pick = (synth.rand_u63(t.numel(), 91, 31, dev()).reshape(t.shape) >> 12) % 2048
            mask = pick < 3
            t[mask] = special[pick[mask]]
        w.tiny_scales_set = True
    A, lg = _inputs(cfg, T, 9100 + T)
    n_flat = T * cfg.top_k
    split = [(st, c) for st in (0, 1) for c in ve.moe_tile_candidates(st) if c[0] == 3]
    assert {st for st, _ in split} == {0, 1}, "no K-split shape among the candidates"
    for st0, c0 in [x for x in split if x[0] == 0]:
        for st1, c1 in [x for x in split if x[0] == 1]:
            ve.moe_tile_set(0, cfg.H, cfg.I, n_flat, c0)
            ve.moe_tile_set(1, cfg.I, cfg.H, n_flat, c1)
            try:
                assert ve.moe_tile_query(0, cfg.H, cfg.I, n_flat) == (c0, True)
                _check(cfg, T, w, A, lg, tight=True)
            finally:
                ve.moe_tile_set(0, cfg.H, cfg.I, n_flat, None)
                ve.moe_tile_set(1, cfg.I, cfg.H, n_flat, None)


def test_k_shared_between_wavefronts_with_rows_outside_the_fast_range():
    """Two tokens, the compiled-in rule's K-split shapes: one row of tiny activations (block
    exponents below the fast path's range) makes its pass take the exact path, which the
    first wavefront of every unit runs over all of K."""
    cfg = synth.MoEConfig("c9", 1536, 1024, 8, 2, (2,), "uniform")
    assert ve.moe_tile_query(0, cfg.H, cfg.I, 4)[0][0] == 3 and ve.moe_tile_query(1, cfg.I, cfg.H, 4)[0][0] == 3
    w = _weights(cfg, 9000)
    A, lg = _inputs(cfg, 2, 9300)
    A = A.copy()
    A[1, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[1, :]) * np.float32(2.0 ** -60))
    g = _run_gpu(cfg, w, A, lg)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw)
    for t in range(2):  # row by row: the rows differ by many orders of magnitude (relative L2 is what binds)
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
    assert np.any(c["out"][1] != 0)


@pytest.mark.parametrize("use_workspace", [True, False])
@pytest.mark.parametrize("bs", [16, 48, 80, 128])
def test_tile_kernels_block_sizes(bs, use_workspace):
    """The tile kernels (more than 512 routed rows) with and without the caller's workspace,
    for block sizes below, above and not dividing their 64- and 128-row groups."""
    cfg = synth.CONFIGS["c1"]
    T, seed = 160, 1700
    w = _weights(cfg, 1500)
    A, lg = _inputs(cfg, T, seed)
    _check(cfg, T, w, A, lg, sample=32, block_size=bs, use_workspace=use_workspace)


@pytest.mark.parametrize("T,use_workspace", [(16, True), (300, True), (300, False)])
def test_expert_map_keeps_local_experts_only(T, use_workspace):
    """Expert parallelism: a rank that owns half the experts (in permuted local order)
    adds only their contributions; selections of the other experts have no sorted row,
    which the combine pass of the workspace path must skip."""
    cfg = synth.CONFIGS["c1"]
    seed = 1800
    w = _weights(cfg, 1500)
    A, lg = _inputs(cfg, T, seed)
    rng = np.random.default_rng(seed)
    local_n = cfg.E // 2
    owned = rng.permutation(cfg.E)[:local_n]
    emap = np.full(cfg.E, -1, dtype=np.int32)
    emap[owned] = np.arange(local_n, dtype=np.int32)
    own = to_dev(owned.astype(np.int64))
    fe = ve.FusedExperts(w.w13[own].contiguous(), w.w13_scale[own].contiguous(),
                         w.w2[own].contiguous(), w.w2_scale[own].contiguous(),
                         expert_map=to_dev(emap), local_num_experts=local_n,
                         scratch=ve.CaptureSafeScratch())
    fe.use_workspace = use_workspace
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    bs = ve.default_block_size(T, cfg.top_k)
    out = fe.apply(to_dev(A, torch.bfloat16), ids, tw, block_size=bs).cpu().numpy()
    ids_np, tw_np = ids.cpu().numpy(), tw.cpu().numpy()
    tw_local = np.where(emap[ids_np] >= 0, tw_np, np.float32(0.0)).astype(np.float32)
    c = cpu_layer(A, w.numpy(), ids_np, tw_local, threads=16)
    max_rel, rel_l2, nf = error_metrics(out, c["out"])
    print(f"c1 T={T} expert map: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL


def test_second_stage_alone_on_the_workspace_path():
    """Small hidden, large intermediate, decode-sized batch: the first stage runs as the
    decode kernel, the second (K = 4096) as the workspace tile kernel, whose split rows
    are then made from act between the stages."""
    cfg = synth.MoEConfig("t", 1024, 4096, 8, 2, (32,), "uniform")
    T, seed = 32, 4200
    w = _weights(cfg, 4200)
    A, lg = _inputs(cfg, T, seed)
    g1, wn = _check(cfg, T, w, A, lg, use_workspace=True)
    g0, _ = _check(cfg, T, w, A, lg, use_workspace=False, weights_np=wn)
    m, l2, nf = error_metrics(g1["out"], g0["out"])
    assert nf and l2 <= 1e-4, (m, l2)


def test_workspace_and_plain_entry_points_agree():
    """Large K (the decode kernel does not apply) at a decode-sized batch: the workspace path
    and the plain entry point compute the same layer."""
    cfg = synth.CONFIGS["c4"]
    T, seed = 24, 4100
    w = _weights(cfg, 4100)
    A, lg = _inputs(cfg, T, seed)
    g1, wn = _check(cfg, T, w, A, lg, use_workspace=True)
    g0, _ = _check(cfg, T, w, A, lg, use_workspace=False, weights_np=wn)
    m, l2, nf = error_metrics(g1["out"], g0["out"])
    assert nf and l2 <= 1e-4, (m, l2)


@pytest.mark.parametrize("T", [8, 200])
def test_accumulate_and_overwrite(T):
    """The ABI accumulates into `out`; VK_HIP_MOE_OVERWRITE_OUT writes it whatever it held."""
    cfg = synth.CONFIGS["c1"]
    w = _weights(cfg, 1500)
    A_bits, lg = _inputs(cfg, T, 1800)
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch())
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    bs = ve.default_block_size(T, cfg.top_k)
    sids, eids, _, max_em = fe.align(ids, bs)
    base = torch.zeros((T, cfg.H), dtype=torch.float32, device=dev())
    fe.fused_call(A, ids, tw, sids, eids, max_em, bs, base)
    acc = torch.full((T, cfg.H), 3.0, dtype=torch.float32, device=dev())
    fe.fused_call(A, ids, tw, sids, eids, max_em, bs, acc)
    over = torch.full((T, cfg.H), float("nan"), dtype=torch.float32, device=dev())
    fe.fused_call(A, ids, tw, sids, eids, max_em, bs, over, overwrite=True)
    torch.cuda.synchronize()
    b = base.cpu().numpy()
    m, l2, nf = error_metrics(acc.cpu().numpy() - 3.0, b)
    assert nf and l2 <= 1e-4, (m, l2)
    m, l2, nf = error_metrics(over.cpu().numpy(), b)
    assert nf and l2 <= 1e-4, (m, l2)


# ---- values outside the fast path's domain ---------------------------------------

def _tiny_case(seed):
    cfg = synth.CONFIGS["c0"]
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    A = synth.make_activations(16, cfg.H, seed)
    lg = synth.make_logits("uniform", 16, cfg.E, seed)
    return cfg, w, A, lg


def _check_columns(g_out, c_out):
    """Column by column: the columns of these cases differ by many orders of magnitude."""
    checked = 0
    for h in range(c_out.shape[1]):
        max_rel, rel_l2, nf = error_metrics(g_out[:, h], c_out[:, h])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (h, max_rel, rel_l2)
        checked += int(np.isfinite(c_out[:, h]).sum())
    return checked


def test_weight_scales_outside_fast_range():
    """Scale bytes outside [64, 190] (and 0xFF, a zero block) take the exact path.  The large
    ones go into the down weights only: through the gate/up product they would overflow."""
    cfg, w, A, lg = _tiny_case(71)
    for t, values in ((w.w13_scale, [0, 1, 2, 63, 255]), (w.w2_scale, [0, 1, 63, 191, 200, 255])):
        special = torch.tensor(values, dtype=torch.uint8, device=dev())
        r = synth.rand_u63(t.numel(), 71, 31, dev()).reshape(t.shape)
        pick = (r >> 12) % 64
        mask = pick < len(values)
        t[mask] = special[pick[mask]]
    g = _run_gpu(cfg, w, A, lg)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw)
    assert _check_columns(g["out"], c["out"]) == c["out"].size  # all finite, all compared


def test_nonfinite_codes():
    """inf and NaN codes in two experts: the tokens routed there get the oracle's non-finite
    outputs position by position, the others stay finite and within tolerance."""
    cfg, w, A, lg = _tiny_case(72)
    r = synth.rand_u63(w.w13[0].numel(), 72, 32, dev()).reshape(w.w13[0].shape)
    w.w13[0][(r >> 10) % 4096 == 0] = 0x6E   # +inf and -inf codes
    r = synth.rand_u63(w.w2[1].numel(), 72, 33, dev()).reshape(w.w2[1].shape)
    w.w2[1][(r >> 10) % 8192 == 0] = 0x7F    # NaN codes
    g, _ = _check(cfg, 16, w, A, lg)
    finite_rows = np.all(np.isfinite(g["out"]), axis=1)
    assert 0 < finite_rows.sum() < 16


def test_activations_outside_fast_range():
    """Huge, tiny and non-finite activations: the pass falls back to the exact path."""
    cfg, w, A, lg = _tiny_case(73)
    A = A.copy()
    A[0, 5] = 0x7F80      # +inf
    A[1, 7] = 0x7FC0      # NaN
    A[2, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[2, :]) * np.float32(2.0 ** 80))
    A[3, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[3, :]) * np.float32(2.0 ** -90))
    A[4, :] = 0
    A[5, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[5, :]) * np.float32(2.0 ** 30))
    g = _run_gpu(cfg, w, A, lg)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw)
    for t in range(16):  # row by row: the rows differ by 50 orders of magnitude
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
    assert np.all(np.isfinite(g["out"][5])) and not np.all(np.isfinite(g["out"][:3]))
