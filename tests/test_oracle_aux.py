"""CPU tests of the oracle's MXFP4 MoE orchestration ops (oracle/aux_oracle.c) against
the reference's own known-answer tests (tests/kernels/moe/test_moe_aux.cpp and
test_moe_aux_fused.cpp, restated), against the compiled reference where it is present
(every bf16 bit pattern as a group's largest value; random groups), and against the
committed fixtures written from the compiled reference."""
from __future__ import annotations

from pathlib import Path

import numpy as np
import pytest

import oracle
from vkernels_amd import synth

GOLDEN = Path(__file__).resolve().parent / "golden"
needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref/libvkref.so not built here")


def _bf(x):
    return synth.f32_to_bf16_bits(np.asarray(x, dtype=np.float32))


def test_quant_round_trip_and_scale_invariant():
    # tests/kernels/moe/test_moe_aux.cpp:73-114
    M, hidden, gs = 4, 64, 32
    repr_ = np.array([0, .25, -.25, 1, -1, 1.5, -1.5, 2, -2, 3, -3, .7, -.7, 2.3, -2.3, .125], np.float32)
    A = _bf(repr_[np.arange(M * hidden) % repr_.size]).reshape(M, hidden)
    packed, scales = oracle.mxfp4_moe_quant(A, gs)
    dq = oracle.mxfp4_dequant_act(packed, scales, gs)
    a = synth.bf16_bits_to_f32(A)
    step = np.where(np.abs(a) <= 0.25, 0.25, 0.5)
    assert np.all(np.isfinite(dq))
    assert np.all(np.abs(np.abs(a) - np.abs(dq)) <= step + 1e-6)
    assert np.all(dq[a == 0] == 0)
    nz = a != 0
    assert np.all((a[nz] < 0) == (dq[nz] < 0))
    sc = (scales.astype(np.uint32) << 23).view(np.float32)
    amax = np.abs(a).reshape(M, hidden // gs, gs).max(axis=2)
    assert np.all(sc >= amax / 3.0 - 1e-6) and np.all(amax / sc <= 3.0 + 1e-6)


def test_quant_zero_group():
    # test_moe_aux.cpp:116-123
    packed, scales = oracle.mxfp4_moe_quant(np.zeros((2, 32), np.uint16), 32)
    assert np.all(scales == 0xFF) and not packed.any()


def test_quant_code_table_and_ties():
    """moe_aux.cpp:62-73: thresholds 0.125 / 0.625 / 1.25 / 1.75 / 2.5, ties to the larger
    magnitude, the sign bit from x < 0."""
    vals = np.array([3.0, 0.124, 0.125, 0.624, 0.625, 1.249, 1.25, 1.749, 1.75, 2.49, 2.5, 2.99,
                     -0.124, -0.125, -0.0, 0.0, -3.0, -1.25], np.float32)
    row = np.zeros(32, np.float32)
    row[:vals.size] = vals
    A = _bf(row).reshape(1, 32)                  # amax = 3 -> scale 1
    packed, scales = oracle.mxfp4_moe_quant(A, 32)
    assert scales[0, 0] == 127
    nib = np.stack([packed[0] & 15, packed[0] >> 4], axis=-1).ravel()
    back = synth.bf16_bits_to_f32(A[0])          # values after the bf16 rounding of the inputs
    want = []
    for x in back[:vals.size]:
        v = abs(float(x))
        mag = 0 if v < .125 else 1 if v < .625 else 2 if v < 1.25 else 3 if v < 1.75 else 4 if v < 2.5 else 5
        want.append(mag | (8 if x < 0 else 0))
    assert list(nib[:vals.size]) == want
    assert nib[12] == 8 and nib[14] == 0         # -0.124 -> code 8 (negative zero), -0.0 -> code 0


def test_sort_gathers_and_scatter_reduce_examples():
    # test_moe_aux.cpp:134-165 and :167-197
    A = np.array([[10, 11, 12, 13], [20, 21, 22, 23], [30, 31, 32, 33]], np.uint16)
    out = oracle.mxfp4_moe_sort(A, [2, 6, 1], 2)
    assert list(out[0]) == [20, 21, 22, 23] and not out[1].any() and list(out[2]) == [10, 11, 12, 13]
    sc = oracle.mxfp4_moe_sort_scales(np.array([[100, 101, 102], [110, 111, 112]], np.uint8), [1, 1, 2], 1)
    assert list(sc[0]) == [110, 111, 112] and list(sc[1]) == [110, 111, 112] and not sc[2].any()
    partial = np.array([[1, 2, 3, 4, 5], [10, 20, 30, 40, 50], [100, 200, 300, 400, 500], [9] * 5], np.float32)
    out = oracle.mxfp4_moe_scatter_reduce(partial, [0.5, 0.5, 1.0, 0.0], [0, 1, 2, 6], 3, 2)
    assert np.allclose(out[0], [5.5, 11, 16.5, 22, 27.5]) and np.allclose(out[1], [100, 200, 300, 400, 500])
    assert not out[2].any()


def test_scatter_reduce_q_matches_float_form_and_passes_nonfinite_codes():
    # test_moe_aux.cpp:199-252
    repr_ = np.array([0, .25, -.25, 1, -1, 1.5, 2, 3], np.float32)
    pf = repr_[np.arange(2 * 32) % repr_.size].reshape(2, 32)
    pq, ps = oracle.mxfp4_moe_quant(_bf(pf), 32)
    out_q = oracle.mxfp4_moe_scatter_reduce_q(pq, ps, [2.0, 0.5], [0, 1], 2, 1, 32)
    out_f = oracle.mxfp4_moe_scatter_reduce(oracle.mxfp4_dequant_act(pq, ps, 32), [2.0, 0.5], [0, 1], 2, 1)
    assert np.array_equal(out_q.view(np.uint32), out_f.view(np.uint32))
    out = oracle.mxfp4_moe_scatter_reduce_q(np.array([[0x76, 0xFE]], np.uint8), np.array([[127]], np.uint8),
                                            [1.0], [0], 1, 1, 4)
    assert out[0, 0] == np.inf and np.isnan(out[0, 1]) and out[0, 2] == -np.inf and np.isnan(out[0, 3])


def test_sorted_quant_is_sort_then_quant():
    """tests/kernels/moe/test_moe_aux_fused.cpp: the fused op equals quant(sort(A)) bit for
    bit, padding rows (ids outside [0, M*top_k), negative ones included) give 0xFF scales and
    zero nibbles, and real rows carry the scales of quant(A) gathered."""
    rng = np.random.default_rng(3)
    M, hidden, top_k, E = 24, 128, 2, 4
    A = synth.make_activations(M, hidden, 91)
    ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
    sids, _, em = oracle.moe_align_block_size(ids, 16, E)
    sids = sids[:em].copy()
    sids[3] = -5
    pk, sc = oracle.mxfp4_moe_sorted_quant(A, sids, top_k)
    pk2, sc2 = oracle.mxfp4_moe_quant(oracle.mxfp4_moe_sort(A, sids, top_k))
    assert np.array_equal(pk, pk2) and np.array_equal(sc, sc2)
    pad = (sids < 0) | (sids >= M * top_k)
    assert np.all(sc[pad] == 0xFF) and not pk[pad].any()
    gathered = oracle.mxfp4_moe_sort_scales(oracle.mxfp4_moe_quant(A)[1], sids, top_k)
    assert np.array_equal(sc[~pad], gathered[~pad])


@needs_ref
def test_quant_every_bf16_pattern_against_the_reference():
    """Every bf16 bit pattern as the only non-zero value of a group (scale byte and its own
    code), and as a member of a group with a larger value."""
    pats = np.arange(65536, dtype=np.uint16)
    A = np.zeros((65536, 32), np.uint16)
    A[:, 5] = pats
    for other in (0, 0x4040, 0x0080, 0x7F00):     # alone; next to 3.0, to the smallest normal, to 2^127
        A[:, 9] = other
        pk, sc = oracle.mxfp4_moe_quant(A)
        rk, rs = oracle.mxfp4_moe_quant(A, use_ref=True)
        assert np.array_equal(sc, rs), other
        assert np.array_equal(pk, rk), other


@needs_ref
def test_aux_ops_against_the_reference_on_random_inputs():
    rng = np.random.default_rng(17)
    M, hidden, top_k, E = 40, 256, 4, 8
    for scale_pow in (0, 60, -60, 120, -125):
        a = synth.bf16_bits_to_f32(synth.make_activations(M, hidden, 92)) * np.float32(2.0 ** scale_pow)
        A = _bf(a).reshape(M, hidden)
        A[0, :32] = 0
        A[1, 7] = 0x7F80
        A[2, 9] = 0x7FC1
        A[3, :] = rng.integers(0, 128, hidden).astype(np.uint16)     # bf16 subnormals
        ids = rng.integers(0, E, (M, top_k)).astype(np.int32)
        sids, _, em = oracle.moe_align_block_size(ids, 16, E)
        sids = sids[:em]
        for fn, args in ((oracle.mxfp4_moe_quant, (A,)), (oracle.mxfp4_moe_sorted_quant, (A, sids, top_k))):
            mine, ref = fn(*args), fn(*args, use_ref=True)
            assert np.array_equal(mine[0], ref[0]) and np.array_equal(mine[1], ref[1]), (fn.__name__, scale_pow)
        assert np.array_equal(oracle.mxfp4_moe_sort(A, sids, top_k), oracle.mxfp4_moe_sort(A, sids, top_k, use_ref=True))
    partial = rng.standard_normal((em, 96)).astype(np.float32)
    tws = rng.random(em).astype(np.float32)
    assert np.array_equal(oracle.mxfp4_moe_scatter_reduce(partial, tws, sids, M, top_k).view(np.uint32),
                          oracle.mxfp4_moe_scatter_reduce(partial, tws, sids, M, top_k, use_ref=True).view(np.uint32))
    pq = rng.integers(0, 256, (em, 48)).astype(np.uint8)
    ps = rng.integers(0, 256, (em, 3)).astype(np.uint8)
    mine = oracle.mxfp4_moe_scatter_reduce_q(pq, ps, tws, sids, M, top_k)
    ref = oracle.mxfp4_moe_scatter_reduce_q(pq, ps, tws, sids, M, top_k, use_ref=True)
    same = (mine == ref) | (np.isnan(mine) & np.isnan(ref))
    assert same.all()


def test_aux_golden_fixture():
    d = np.load(GOLDEN / "aux_quant.npz")
    A = d["A"]
    pk, sc = oracle.mxfp4_moe_quant(A)
    assert np.array_equal(pk, d["packed"]) and np.array_equal(sc, d["scales"])
    spk, ssc = oracle.mxfp4_moe_sorted_quant(A, d["sorted_ids"], int(d["top_k"]))
    assert np.array_equal(spk, d["sorted_packed"]) and np.array_equal(ssc, d["sorted_scales"])
    out = oracle.mxfp4_moe_scatter_reduce(d["partial"], d["topk_w_sorted"], d["sorted_ids"], A.shape[0], int(d["top_k"]))
    assert np.array_equal(out.view(np.uint32), d["reduced"].view(np.uint32))
    table = d["scale_table"]                      # scale byte of every positive bf16 pattern
    mine = np.array([oracle.aux_scale_byte(b) for b in range(32768)], dtype=np.uint8)
    assert np.array_equal(mine, table)


def test_act_model_one_term_is_quant_then_dequant():
    bits = synth.make_activations(8, 64, 93)
    oracle_vals = np.stack([oracle.act_model_block32(b, 1) for b in bits.reshape(-1, 32)]).reshape(8, 64)
    pk, sc = oracle.mxfp4_moe_quant(bits)
    assert np.array_equal(oracle_vals, oracle.mxfp4_dequant_act(pk, sc))
