"""Writes tests/golden/*.npz: outputs of the REFERENCE's own moe_fused.cpp
(built by oracle/Makefile target `ref` into oracle/_ref/libvkref.so) on seeded
inputs, so that the oracle restatement can be checked against the reference
on machines that do not have the reference tree.

    python tests/golden/make_golden.py

Only data is stored: the seeds / small input tensors and the reference's
outputs.  Needs oracle/_ref/libvkref.so (run `make -C oracle ref` where
/root/reference is mounted).
"""
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

import oracle  # noqa: E402
from vkernels_amd import synth  # noqa: E402

OUT = Path(__file__).resolve().parent


def layer_case(name, cfg, T, seed, **kw):
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed).numpy()
    A = synth.make_activations(T, cfg.H, seed)
    lg = synth.make_logits(cfg.logits, T, cfg.E, seed, A, cfg.H)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)   # routing is an input here
    sids, eids, em = oracle.moe_align_block_size(ids, 16, cfg.E, use_ref=True)
    tws = oracle.gather_sorted_weights(tw, sids[:em])
    b13 = b2 = None
    if kw.pop("bias", False):
        b13 = synth.rand_normal((cfg.E, 2 * cfg.I), seed, 21).astype(np.float32)
        b2 = synth.rand_normal((cfg.E, cfg.H), seed, 22).astype(np.float32)
    out, act = oracle.fused_moe_mxfp4(A, *w, sids, tws, eids, T, cfg.H, cfg.I, cfg.top_k, em,
                                      b13=b13, b2=b2, use_ref=True, **kw)
    np.savez_compressed(OUT / f"{name}.npz", seed=seed, T=T, cfg=cfg.name, topk_ids=ids, topk_w=tw,
                        sorted_ids=sids[:em], expert_ids=eids[:em // 16], EM=em,
                        out=out, act=act[:em], kw=np.array(json.dumps(kw)),
                        bias=b13 is not None,
                        checksum_inputs=np.array([int(A.astype(np.uint64).sum()),
                                                  int(w[0].astype(np.uint64).sum()),
                                                  int(w[2].astype(np.uint64).sum())]))
    print(name, "EM", em, "out rms", float(np.sqrt(np.mean(out.astype(np.float64) ** 2))))


def main():
    if not oracle.have_ref():
        raise SystemExit("oracle/_ref/libvkref.so missing: run `make -C oracle ref`")
    c0 = synth.CONFIGS["c0"]
    layer_case("c0_T16_swiglu", c0, 16, synth.config_seed(c0, 16))
    layer_case("c0_T16_swiglu_limit_bias", c0, 16, 4242, swiglu_limit=7.0, bias=True)
    layer_case("c0_T16_situ_bias", c0, 16, 4343, activation=1, beta=4.0, linear_beta=25.0, bias=True)
    small = synth.MoEConfig("c9", 128, 64, 4, 2, (5,), "uniform")
    layer_case("small_T5", small, 5, 77)

    # dequant table: all 16 codes x all 256 scale bytes, reference's LUT path
    packed = np.zeros((64, 32), dtype=np.uint8)
    codes = np.arange(16, dtype=np.uint8)
    packed[:] = (codes[np.arange(32) % 16] | (codes[(np.arange(32) + 5) % 16] << 4))[None, :]
    table = np.zeros((256, 16), dtype=np.uint16)
    for s in range(256):
        scale = np.full((64, 2), s, dtype=np.uint8)
        t = oracle.dequant_weight_tile(packed, scale, 64, 64, use_ref=True)
        for kp in range(16):
            table[s, kp] = t[2 * kp, 0]          # low nibble of byte kp = code kp
    np.savez_compressed(OUT / "dequant_table.npz", table=table)
    print("dequant table", table.shape)

    # align cases
    rng = np.random.default_rng(5)
    cases = {}
    for i, (M, k, E, bs) in enumerate([(8, 4, 4, 16), (17, 2, 8, 64), (64, 8, 256, 16),
                                       (5, 16, 256, 64), (33, 1, 7, 32), (3, 2, 4, 16)]):
        ids = rng.integers(-1 if i == 5 else 0, E + (1 if i == 5 else 0), (M, k)).astype(np.int32)
        s, e, em = oracle.moe_align_block_size(ids, bs, E, use_ref=True)
        cases[f"ids{i}"] = ids
        cases[f"meta{i}"] = np.array([M, k, E, bs, em])
        cases[f"sids{i}"] = s[:em]
        cases[f"eids{i}"] = e[:em // bs]
    np.savez_compressed(OUT / "align_cases.npz", n=6, **cases)
    print("align cases written")

    # moe_aux.cpp: activation quantisation (token and sorted order), routed combine, and the
    # scale byte of every positive bf16 pattern as a group's largest value
    M, hidden, top_k, E = 12, 128, 2, 4
    A = synth.make_activations(M, hidden, 95)
    A[0, :32] = 0
    A[1, 40] = 0x7F80
    A[2, :] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(A[2, :]) * np.float32(2.0 ** -100))
    ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
    sids, _, em = oracle.moe_align_block_size(ids, 16, E, use_ref=True)
    sids = sids[:em]
    packed, scales = oracle.mxfp4_moe_quant(A, use_ref=True)
    spk, ssc = oracle.mxfp4_moe_sorted_quant(A, sids, top_k, use_ref=True)
    partial = rng.standard_normal((em, 64)).astype(np.float32)
    tws = rng.random(em).astype(np.float32)
    reduced = oracle.mxfp4_moe_scatter_reduce(partial, tws, sids, M, top_k, use_ref=True)
    pats = np.zeros((32768, 32), dtype=np.uint16)
    pats[:, 0] = np.arange(32768, dtype=np.uint16)
    scale_table = oracle.mxfp4_moe_quant(pats, use_ref=True)[1][:, 0]
    np.savez_compressed(OUT / "aux_quant.npz", A=A, top_k=top_k, sorted_ids=sids, packed=packed,
                        scales=scales, sorted_packed=spk, sorted_scales=ssc, partial=partial,
                        topk_w_sorted=tws, reduced=reduced, scale_table=scale_table)
    print("aux fixture written, EM", em)


if __name__ == "__main__":
    main()
