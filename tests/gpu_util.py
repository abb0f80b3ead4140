"""Shared helpers of the GPU parity tests: run the layer through the C ABI on
torch device tensors and through the CPU oracle on the same inputs."""
from __future__ import annotations

import ctypes

import numpy as np
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

# Tolerances of the layer output (bf16 activations, fp32 accumulation).
#
# The synthetic layers produce outputs with an RMS of 1e4..1e6, where one fp32
# ulp is already 1e-3..6e-2, and individual elements are sums of terms that
# cancel; a different (equally valid) summation order alone moves such an
# element by more than 2e-2 absolute.  "max-abs error <= 2e-2" is therefore
# measured in units of the output's scale: for every element,
# |gpu - cpu| / max(|cpu|, rms(cpu), 1) -- relative for the elements that stand
# above the RMS (with block scales of 2^+-20 a few outputs are hundreds of
# times the RMS), RMS-relative for the ones below it.  The element-wise figure
# of the reference's own harness, |gpu - cpu| / max(|cpu|, 1)
# (meta/benchmarks/test_moe_fused_correct.hip:195-214), is reported next to it.
MAX_ABS_TOL = 2e-2   # max |gpu - cpu| / max(|cpu|, rms(cpu), 1)
REL_L2_TOL = 5e-3    # ||gpu - cpu||_2 / ||cpu||_2


def dev():
    return torch.device("cuda", 0)


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.to(dev())


def error_metrics(gpu: np.ndarray, cpu: np.ndarray):
    """(scaled max-abs error, relative L2 error, non-finite entries agree)."""
    g = gpu.astype(np.float64).ravel()
    c = cpu.astype(np.float64).ravel()
    finite = np.isfinite(c)
    gn, cn = g[~finite], c[~finite]
    same_nonfinite = bool(np.array_equal(np.isnan(gn), np.isnan(cn)) and
                          np.array_equal(gn[~np.isnan(gn)], cn[~np.isnan(cn)]))
    g, c = g[finite], c[finite]
    if g.size == 0:
        return 0.0, 0.0, same_nonfinite
    if not np.all(np.isfinite(g)):
        return float("inf"), float("inf"), False
    rms = float(np.sqrt(np.mean(c * c)))
    max_abs = float(np.max(np.abs(g - c) / np.maximum(np.abs(c), max(rms, 1.0))))
    denom = float(np.linalg.norm(c))
    rel_l2 = float(np.linalg.norm(g - c) / denom) if denom > 0 else float(np.linalg.norm(g - c))
    return max_abs, rel_l2, same_nonfinite


def elementwise_max_rel(gpu, cpu):
    g = gpu.astype(np.float64).ravel()
    c = cpu.astype(np.float64).ravel()
    ok = np.isfinite(c) & np.isfinite(g)
    return float(np.max(np.abs(g[ok] - c[ok]) / np.maximum(np.abs(c[ok]), 1.0))) if ok.any() else 0.0


def gpu_layer(A_bits, weights, topk_ids=None, topk_w=None, logits=None, top_k=None,
              block_size=None, **kw):
    """Run (router ->) align -> fused layer on the GPU.  Returns numpy results."""
    w13, w13s, w2, w2s = (t if isinstance(t, torch.Tensor) else to_dev(t) for t in weights)
    fe = ve.FusedExperts(w13.to(dev()), w13s.to(dev()), w2.to(dev()), w2s.to(dev()),
                         scratch=ve.CaptureSafeScratch(), **kw)
    A = to_dev(A_bits, torch.bfloat16)
    if logits is not None:
        ids, w = fe.route(to_dev(logits), top_k, True)
    else:
        ids = to_dev(topk_ids.astype(np.int32))
        w = None if topk_w is None else to_dev(topk_w.astype(np.float32))
    M = A.shape[0]
    bs = ve.default_block_size(M) if block_size is None else block_size
    sids, eids, out_em, max_em = fe.align(ids, bs)
    out = fe.apply(A, ids, w, block_size=bs)
    torch.cuda.synchronize()
    act = fe.scratch.get(("act", fe.ispp), max_em * fe.ispp, dtype=torch.bfloat16, device=dev())
    return dict(out=out.cpu().numpy(), topk_ids=ids.cpu().numpy(),
                topk_w=None if w is None else w.cpu().numpy(),
                sorted_ids=sids.cpu().numpy(), expert_ids=eids.cpu().numpy(),
                EM=int(out_em.cpu().item()), max_EM=max_em, block_size=bs,
                act=act.view(torch.int16).cpu().numpy().view(np.uint16).reshape(max_em, fe.ispp))


def cpu_layer(A_bits, weights_np, topk_ids, topk_w, block_size=16, threads=8, **kw):
    """The oracle on given routing.  block_size only changes the row layout."""
    oracle.set_threads(threads)
    M, hidden = A_bits.shape
    E = weights_np[0].shape[0]
    ispp = weights_np[0].shape[1] // 2
    top_k = topk_ids.shape[1]
    sids, eids, em = oracle.moe_align_block_size(topk_ids, 16, E)
    tws = oracle.gather_sorted_weights(topk_w, sids[:max(em, 1)])
    out, act = oracle.fused_moe_mxfp4(A_bits, *weights_np, sids, tws, eids, M, hidden, ispp,
                                      top_k, em, **kw)
    return dict(out=out, act=act[:em], sorted_ids=sids[:em], expert_ids=eids[:em // 16], EM=em)


def make_case(cfg: synth.MoEConfig, T: int, seed=None):
    seed = synth.config_seed(cfg, T) if seed is None else seed
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed)
    A = synth.make_activations(T, cfg.H, seed)
    lg = synth.make_logits(cfg.logits, T, cfg.E, seed, A, cfg.H)
    return A, lg, w


# The scaled-MFMA paths that split the activations exactly (decode kernels, tile kernels
# on raw weights) differ from the oracle by the order of the fp32 sums only; measured
# 6e-6 .. 1.8e-4 relative L2 and up to 6e-3 of the RMS for the worst element (sums that
# cancel).  These tighter bounds are asserted for them next to the contract's, so that a
# regression of a factor of a few is noticed.
EXACT_SPLIT_MAX_ABS_TOL = 1e-2
EXACT_SPLIT_REL_L2_TOL = 5e-4


def literal_max_rel(gpu, cpu):
    """The reference harness's own figure: max |gpu - cpu| / max(|cpu|, 1)
    (meta/benchmarks/test_moe_fused_correct.hip:195-214)."""
    return elementwise_max_rel(gpu, cpu)


def edge_tokens(g, n_flat, top_k, want, seed):
    """Tokens whose sorted rows sit where a tile kernel breaks: first and last routed row
    of windows of 128, rows either side of 32-row tile boundaries, the last row of an
    expert's segment, rows of the most and the least popular expert; then random ones."""
    sids, eids, bs = g["sids"], g["eids"], g["bs"]
    routed = np.nonzero(sids < n_flat)[0]
    rows = set()
    win = routed // 128
    first = routed[np.r_[True, win[1:] != win[:-1]]]
    last = routed[np.r_[win[1:] != win[:-1], True]]
    rng = np.random.default_rng(seed)
    for arr in (first, last):
        rows.update(rng.choice(arr, min(arr.size, 24), replace=False).tolist())
    edge = routed[np.isin(routed % 32, (0, 31))]
    rows.update(rng.choice(edge, min(edge.size, 24), replace=False).tolist())
    expert_of_row = np.repeat(eids, bs)[routed]
    counts = np.bincount(expert_of_row[expert_of_row >= 0])
    live = np.nonzero(counts)[0]
    for e in (live[np.argmax(counts[live])], live[np.argmin(counts[live])]):
        er = routed[expert_of_row == e]
        rows.update(er[[0, -1]].tolist())
    tokens = set((sids[list(rows)] // top_k).tolist())
    T = n_flat // top_k
    extra = rng.permutation(T)
    for t in extra:
        if len(tokens) >= want:
            break
        tokens.add(int(t))
    return np.sort(np.fromiter(tokens, dtype=np.int64))
