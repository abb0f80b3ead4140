"""The decode kernel that holds the rows a chunk of K at a time (prepacked form): rows of
any K, and blocks of 32 rows whose two 16-row tiles share one pass over the expert's
weights.  Checked against the oracle like every other call, and against the same call in
blocks of 16 on the resident decode kernel: both walk the K steps of a weight row in order
and add the same two products a step, so the first stage's output is the same bits row for
row."""
from __future__ import annotations

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
CHUNKED = 4


def _act_by_flat_row(g, n_flat):
    rows = np.nonzero(g["sids"] < n_flat)[0]
    order = np.argsort(g["sids"][rows])
    assert np.array_equal(g["sids"][rows][order], np.arange(n_flat))
    return g["act"][rows][order]


@pytest.mark.parametrize("name,T", [("c0", 16), ("c1", 64), ("c2", 64), ("c4", 33), ("c4", 100), ("c4", 255),
                                    ("c1", 200)])
def test_blocks_of_32_rows_in_one_pass(name, T):
    cfg = synth.CONFIGS[name]
    n_flat = T * cfg.top_k
    for stage, (K, ncols) in enumerate(((cfg.H, cfg.I), (cfg.I, cfg.H))):
        # (beyond 512 rows the range follows the rows per expert, which the query does not know)
        shape, _ = ve.moe_tile_query(stage, K, ncols, min(n_flat, 512), packed=True, block_size=32)
        assert shape[0] == CHUNKED, (stage, shape)
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6600 + T)
    g, wn = cfgs._check(cfg, T, w, A, lg, gpu_kw=PACKED_ONLY, tight=True, block_size=32,
                        stagewise=(name == "c4"))
    counts = np.bincount(g["ids"].ravel(), minlength=cfg.E)
    print(f"{name} T={T}: rows per expert up to {counts.max()}, experts with 17 to 32 rows: "
          f"{int(((counts > 16) & (counts <= 32)).sum())}")
    if n_flat <= 512:   # the same call in blocks of 16 is the resident kernel's
        b = cfgs._run_gpu(cfg, w, A, lg, 16, None, **PACKED_ONLY)
        assert np.array_equal(_act_by_flat_row(g, n_flat), _act_by_flat_row(b, n_flat)), \
            "the first stage differs from the resident kernel's"
        m, l2, nf = error_metrics(g["out"], b["out"])
        assert nf and l2 <= 1e-5, (m, l2)


@pytest.mark.parametrize("H,I,E,k,T", [(4608, 256, 4, 2, 5), (7168, 2048, 16, 4, 3), (7168, 2048, 16, 4, 40),
                                       (512, 4224, 4, 2, 9), (8192, 128, 8, 2, 17)])
@pytest.mark.parametrize("bs", [16, 32])
def test_rows_of_any_K(H, I, E, k, T, bs):
    """Rows of more than 4096 values (first stage) or 3072 (second stage): the resident kernel
    cannot hold them; the chunked kernel takes them on the prepacked form, without the raw
    tensors and without a workspace."""
    cfg = synth.MoEConfig("wide", H, I, E, k, (T,), "uniform")
    seed = 6700 + T
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    A, lg = cfgs._inputs(cfg, T, seed)
    shape, _ = ve.moe_tile_query(0 if H > 4096 else 1, max(H, I), min(H, I), T * k, packed=True, block_size=bs)
    assert shape[0] == CHUNKED, shape
    g = cfgs._run_gpu(cfg, w, A, lg, bs, None, **PACKED_ONLY)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    max_rel, rel_l2, nf = error_metrics(g["out"], c["out"])
    print(f"{H}x{I}x{E}x{k} T={T} bs={bs}: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL


@pytest.mark.parametrize("bs", [16, 32])
def test_values_outside_the_range_on_the_chunked_kernel(bs):
    """inf/NaN codes and out-of-range scale bytes (flagged units) and rows with inf, NaN, huge
    and tiny values (marked segments) take the exact path, a unit at a time, as on the
    resident kernel.  Rows of 4608 values, so that the first stage is the chunked kernel's at
    either block size."""
    cfg = synth.MoEConfig("t", 4608, 512, 8, 2, (24,), "uniform")
    T, seed = 24, 6800
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    r = synth.rand_u63(w.w13[0].numel(), seed, 32, dev()).reshape(w.w13[0].shape)
    w.w13[0][(r >> 10) % 65536 == 0] = 0x6E
    r = synth.rand_u63(w.w2[1].numel(), seed, 33, dev()).reshape(w.w2[1].shape)
    w.w2[1][(r >> 10) % 8192 == 0] = 0x7F
    w.w2_scale[2][::7, 1] = 200
    w.w13_scale[3][::5, 0] = 2
    A, lg = cfgs._inputs(cfg, T, seed)
    A = A.copy()
    A[0, 5] = 0x7F80
    A[1, 4200] = 0x7FC0
    A[2, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[2, :]) * np.float32(2.0 ** 80))
    A[3, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[3, :]) * np.float32(2.0 ** -90))
    lg = lg.copy()
    lg[:, :4] += 4.0
    g = cfgs._run_gpu(cfg, w, A, lg, bs, None, **PACKED_ONLY)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    for t in range(T):   # row by row: the rows differ by many orders of magnitude
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
    assert np.bincount(ids.ravel(), minlength=cfg.E)[:4].min() > 0


def test_one_expert_takes_every_row_in_blocks_of_32():
    """All tokens on one expert (runs of the same expert side by side), the others empty."""
    cfg = synth.CONFIGS["c4"]
    T = 40
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 6900)
    lg = lg.copy()
    lg[:, 7] += 30.0
    g, _ = cfgs._check(cfg, T, w, A, lg, gpu_kw=PACKED_ONLY, block_size=32, stagewise=True)
    assert np.bincount(g["ids"].ravel(), minlength=cfg.E)[7] == T


@pytest.mark.parametrize("variant", ["bias_limit", "situ_bias"])
def test_epilogues_on_the_chunked_kernel(variant):
    """Biases, the clamp and SiTU through the chunked kernel's calls of the shared epilogue."""
    cfg = synth.CONFIGS["c1"]
    T, seed = 48, 1500
    w = cfgs._weights(cfg, seed)
    A, lg = cfgs._inputs(cfg, T, seed)
    b13 = (synth.rand_normal((cfg.E, 2 * cfg.I), seed, 21) * 0.5).astype(np.float32)
    b2 = (synth.rand_normal((cfg.E, cfg.H), seed, 22) * 0.5).astype(np.float32)
    gpu_kw, cpu_kw = dict(PACKED_ONLY, b13=to_dev(b13), b2=to_dev(b2)), dict(b13=b13, b2=b2)
    if variant == "bias_limit":
        gpu_kw.update(swiglu_limit=1.5)
        cpu_kw.update(swiglu_limit=1.5)
    else:
        gpu_kw.update(activation="situ", beta=3.0, linear_beta=20.0)
        cpu_kw.update(activation=1, beta=3.0, linear_beta=20.0)
    cfgs._check(cfg, T, w, A, lg, gpu_kw=gpu_kw, cpu_kw=cpu_kw, block_size=32)


@pytest.mark.parametrize("name,T", [("c4", 33), ("c1", 64)])
def test_chunked_shapes_forced_in_blocks_of_16(name, T):
    """The tuning store may name the chunked kernel for calls the rules give to the resident
    one: blocks of 16, a tile a pass (second stage of c4: rows of 1536 values, its
    single-chunk form)."""
    cfg = synth.CONFIGS[name]
    n_flat = T * cfg.top_k
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 7000 + T)
    keys = ((0, cfg.H, cfg.I), (1, cfg.I, cfg.H))
    try:
        for stage, K, ncols in keys:
            ve.moe_tile_set(stage, K, ncols, n_flat, (CHUNKED, 8, 2, 2) if stage == 0 else (CHUNKED, 8, 1, 4))
        g, _ = cfgs._check(cfg, T, w, A, lg, gpu_kw=PACKED_ONLY, tight=True, block_size=16, stagewise=(name == "c4"))
    finally:
        for stage, K, ncols in keys:
            ve.moe_tile_set(stage, K, ncols, n_flat, None)
    b = cfgs._run_gpu(cfg, w, A, lg, 16, None, **PACKED_ONLY)
    assert np.array_equal(_act_by_flat_row(g, n_flat), _act_by_flat_row(b, n_flat))
    m, l2, nf = error_metrics(g["out"], b["out"])
    assert nf and l2 <= 1e-5, (m, l2)


def test_more_runs_than_workgroups():
    """384 experts, 800 routed rows in blocks of 32: more runs (blocks with rows) than the launch
    has workgroups, so the (run, unit) space is cut evenly and a workgroup's slice spans runs,
    segment after segment with different rows."""
    cfg = synth.MoEConfig("many", 256, 128, 384, 4, (200,), "uniform")
    T, seed = 200, 7100
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed, device=dev())
    A, lg = cfgs._inputs(cfg, T, seed)
    g = cfgs._run_gpu(cfg, w, A, lg, 32, None, **PACKED_ONLY)
    runs = int((g["eids"] >= 0).sum())
    assert runs > 304, runs       # (more than the compute units of the device)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    max_rel, rel_l2, nf = error_metrics(g["out"], c["out"])
    print(f"{runs} runs: max_abs/rms={max_rel:.3e} rel_l2={rel_l2:.3e}")
    assert nf and max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL
