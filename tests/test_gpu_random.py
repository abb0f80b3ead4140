"""Randomised parity of small layers: shapes, block sizes, routing skew and the weight
path drawn at random (fixed seeds), router and alignment through the one-call entry
point compared bit for bit, the layer within the contract's tolerances.  Small shapes
reach corners the benchmark configurations do not: one or two experts, top_k = E,
sums of 64 products, blocks of 128 rows holding a single routed row."""
from __future__ import annotations

import numpy as np
import pytest
import torch

import oracle
from vkernels_amd import synth
from vkernels_amd import vllm_experts as ve

from gpu_util import MAX_ABS_TOL, REL_L2_TOL, cpu_layer, dev, error_metrics, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [1, 7])
def test_random_small_layers(seed):
    rng = np.random.default_rng(seed)
    worst = [0.0, 0.0]
    for case in range(24):
        E = int(rng.choice([2, 4, 8, 17, 32, 64, 100, 128, 256]))
        k = int(rng.integers(1, min(8, E) + 1))
        H = int(rng.choice([64, 128, 256, 512, 1024, 2880]))
        I = int(rng.choice([64, 128, 256, 512, 1024]))
        T = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 31, 40, 64, 96, 128, 150, 200]))
        bs = int(rng.choice([16, 16, 16, 32, 64, 128]))
        kind = str(rng.choice(["uniform", "zipf", "router"]))
        prepack = bool(rng.integers(0, 2))
        s = int(rng.integers(1, 1 << 30))
        what = dict(case=case, E=E, k=k, H=H, I=I, T=T, bs=bs, routing=kind, prepack=prepack, seed=s)
        print(what, flush=True)
        w = synth.make_weights(E, H, I, s, device=dev())
        A_bits = synth.make_activations(T, H, s)
        lg = synth.make_logits(kind, T, E, s, A_bits, H)
        fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(),
                             prepack=prepack)
        ids, tw, sids, eids, out_em, max_em, _ = fe.route_align(to_dev(lg), k, True, bs)
        out = fe.apply(to_dev(A_bits, torch.bfloat16), ids, tw, block_size=bs, aligned=(sids, eids, max_em))
        torch.cuda.synchronize()
        rid, rw = oracle.route_topk(lg, k, True)
        assert np.array_equal(ids.cpu().numpy(), rid), what
        assert np.array_equal(tw.cpu().numpy().view(np.uint32), rw.view(np.uint32)), what
        rs, re_, rem = oracle.moe_align_block_size_with_map(rid.ravel(), E, bs, None, max_EM=max_em)
        assert int(out_em.item()) == rem, what
        assert np.array_equal(sids.cpu().numpy(), rs) and np.array_equal(eids.cpu().numpy(), re_), what
        c = cpu_layer(A_bits, w.numpy(), rid, rw, threads=16)
        m, l2, nf = error_metrics(out.cpu().numpy(), c["out"])
        assert nf and m <= MAX_ABS_TOL and l2 <= REL_L2_TOL, (what, m, l2)
        worst = [max(worst[0], m), max(worst[1], l2)]
    print(f"seed {seed}: worst max_abs/rms={worst[0]:.3e} rel_l2={worst[1]:.3e}")
    # measured: 1e-2 / 8e-4 at most; the contract is 2e-2 / 5e-3
    assert worst[0] <= 1.2e-2 and worst[1] <= 1.5e-3


def test_random_layers_on_the_chunked_decode_kernel():
    """The same on the prepacked form alone, drawn where the chunked decode kernel runs: blocks
    of 32 rows at any width, or blocks of 16 with rows the resident kernel cannot hold (more than
    4096 values in the first stage, more than 3072 in the second)."""
    rng = np.random.default_rng(11)
    worst = [0.0, 0.0]
    for case in range(24):
        E = int(rng.choice([2, 4, 8, 17, 32, 64, 128]))
        k = int(rng.integers(1, min(8, E) + 1))
        bs = int(rng.choice([16, 32, 32, 32]))
        if bs == 16:
            H, I = [(4160, 128), (5120, 256), (256, 3136), (4608, 3200)][int(rng.integers(0, 4))]
        else:
            H = int(rng.choice([64, 128, 512, 1024, 2880, 4160]))
            I = int(rng.choice([64, 256, 512, 1024, 3136]))
        T = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 31, 40, 64, 96, 128]))
        kind = str(rng.choice(["uniform", "zipf", "router"]))
        s = int(rng.integers(1, 1 << 30))
        what = dict(case=case, E=E, k=k, H=H, I=I, T=T, bs=bs, routing=kind, seed=s)
        print(what, flush=True)
        stages = [ve.moe_tile_query(st, K, n, min(T * k, 512), packed=True, block_size=bs)[0][0]
                  for st, K, n in ((0, H, I), (1, I, H))]
        assert 4 in stages, (what, stages)     # at least one stage is the chunked kernel's
        w = synth.make_weights(E, H, I, s, device=dev())
        A_bits = synth.make_activations(T, H, s)
        lg = synth.make_logits(kind, T, E, s, A_bits, H)
        wn = w.numpy()
        fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(),
                             prepack=True, keep_raw=False)
        del w
        ids, tw, sids, eids, out_em, max_em, _ = fe.route_align(to_dev(lg), k, True, bs)
        out = fe.apply(to_dev(A_bits, torch.bfloat16), ids, tw, block_size=bs, aligned=(sids, eids, max_em))
        torch.cuda.synchronize()
        rid, rw = oracle.route_topk(lg, k, True)
        assert np.array_equal(ids.cpu().numpy(), rid), what
        c = cpu_layer(A_bits, wn, rid, rw, threads=16)
        m, l2, nf = error_metrics(out.cpu().numpy(), c["out"])
        assert nf and m <= MAX_ABS_TOL and l2 <= REL_L2_TOL, (what, m, l2)
        worst = [max(worst[0], m), max(worst[1], l2)]
    print(f"chunked kernel: worst max_abs/rms={worst[0]:.3e} rel_l2={worst[1]:.3e}")
    assert worst[0] <= 1.2e-2 and worst[1] <= 1.5e-3
