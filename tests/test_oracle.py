"""Pins the CPU oracle (oracle/) before anything is compared against it.

Sources of truth, in this order:
  * the known-answer tests of the reference's own unit tests
    (tests/kernels/moe/test_moe_fused.cpp, test_moe_align_oracle.cpp,
    tests/kernels/moe/test_moe.cpp, tests/capi/test_capi.cpp) restated here
    with the same inputs and expectations;
  * golden fixtures under tests/golden/ produced by a build of the reference's
    moe_fused.cpp (tests/golden/make_golden.py);
  * the live reference build oracle/_ref/libvkref.so, when present;
  * for the router, which has no reference CPU code: closed forms, brute
    force, invariants and torch's softmax/topk as an independent library.
"""
import json
import math
from pathlib import Path

import numpy as np
import pytest

import oracle
from vkernels_amd import synth

GOLDEN = Path(__file__).resolve().parent / "golden"


def f2bf(v):
    return int(synth.f32_to_bf16_bits(np.array([v], dtype=np.float32))[0])


def bf2f(b):
    return synth.bf16_bits_to_f32(np.asarray(b, dtype=np.uint16))


E2M1 = {0.0: 0, 0.25: 1, 1.0: 2, 1.5: 3, 2.0: 4, 3.0: 5}


def pack_pair(v0, v1):
    def nib(v):
        return E2M1[abs(v)] | (8 if v < 0 else 0)
    return nib(v0) | (nib(v1) << 4)


# --------------------------------------------------------------------------
# scalar decoders
# --------------------------------------------------------------------------

def test_nibble_table_known_answers():
    # tests/kernels/moe/test_moe.cpp:76-190 and moe_fused.cpp:24-39
    expect = [0.0, 0.25, 1.0, 1.5, 2.0, 3.0, math.inf, math.nan]
    for code in range(16):
        bits = oracle.fp4nib_to_f32bits(code)
        val = np.array([bits], dtype=np.uint32).view(np.float32)[0]
        mag = expect[code & 7]
        if math.isnan(mag):
            assert bits == 0x7FC00000  # NaN carries no sign
        else:
            assert val == (-mag if code & 8 else mag)
            assert (bits >> 31) == (code >> 3)  # -0 keeps its sign


def test_ue8m0_known_answers():
    assert oracle.ue8m0_to_float(0xFF) == 0.0
    assert oracle.ue8m0_to_float(127) == 1.0
    assert oracle.ue8m0_to_float(128) == 2.0
    assert oracle.ue8m0_to_float(1) == 2.0 ** -126
    assert oracle.ue8m0_to_float(0) == 2.0 ** -127
    assert oracle.ue8m0_to_float(254) == 2.0 ** 127


def test_bf16_rounding_rule():
    assert oracle.f32bits_to_bf16(0x3F800000) == 0x3F80
    assert oracle.f32bits_to_bf16(0x3F808000) == 0x3F80      # tie -> even
    assert oracle.f32bits_to_bf16(0x3F818000) == 0x3F82      # tie -> even (up)
    assert oracle.f32bits_to_bf16(0x3F808001) == 0x3F81
    assert oracle.f32bits_to_bf16(0x7FC00000) == 0x7FC0      # NaN not special-cased


# --------------------------------------------------------------------------
# dequant
# --------------------------------------------------------------------------

def test_dequant_matches_golden_table():
    table = np.load(GOLDEN / "dequant_table.npz")["table"]
    packed = np.zeros((64, 32), dtype=np.uint8)
    codes = np.arange(16, dtype=np.uint8)
    packed[:] = (codes[np.arange(32) % 16] | (codes[(np.arange(32) + 5) % 16] << 4))[None, :]
    for s in range(256):
        t = oracle.dequant_weight_tile(packed, np.full((64, 2), s, np.uint8), 64, 64)
        assert np.array_equal(t[0:32:2, 0], table[s])


def test_dequant_closed_form_finite():
    """bf16(code value * 2^(s-127)) is exact for finite codes and mid scales."""
    vals = np.array([0, .25, 1, 1.5, 2, 3], dtype=np.float64)
    packed = np.array([[c | (c << 4) for c in synth.FINITE_CODES] * 3][0][:32], dtype=np.uint8)[None, :]
    packed = np.repeat(packed, 4, axis=0)
    for s in (100, 123, 127, 129, 150):
        t = bf2f(oracle.dequant_weight_tile(packed, np.full((4, 2), s, np.uint8), 4, 64))
        for kp in range(32):
            c = packed[0, kp] & 15
            want = vals[c & 7] * (-1 if c & 8 else 1) * 2.0 ** (s - 127)
            assert t[2 * kp, 0] == want and t[2 * kp + 1, 0] == want


def test_dequant_lut_equals_per_byte_everywhere():
    # tests/kernels/moe/test_moe_fused.cpp:591-621
    N = K = 64
    packed = ((np.arange(N * K // 2) & 0xFF).astype(np.uint8)).reshape(N, K // 2)
    for s in range(256):
        scale = np.full((N, K // 32), s, np.uint8)
        a = oracle.dequant_weight_tile(packed, scale, N, K, which="lut")
        b = oracle.dequant_weight_tile(packed, scale, N, K, which="ref")
        assert np.array_equal(a, b)


def test_dequant_varying_scales_and_strides():
    # tests/kernels/moe/test_moe_fused.cpp:629-656, plus strided sources
    rng = np.random.default_rng(1)
    for _ in range(50):
        packed = rng.integers(0, 256, (64, 48), dtype=np.uint8)   # row stride 48 > K/2
        scale = rng.integers(0, 256, (64, 5), dtype=np.uint8)
        a = oracle.dequant_weight_tile(packed, scale, 64, 64, stride_packed=48, stride_scale_n=5,
                                       which="lut")
        b = oracle.dequant_weight_tile(packed, scale, 64, 64, stride_packed=48, stride_scale_n=5,
                                       which="ref")
        assert np.array_equal(a, b)
        if oracle.have_ref():
            c = oracle.dequant_weight_tile(packed, scale, 64, 64, stride_packed=48,
                                           stride_scale_n=5, use_ref=True)
            assert np.array_equal(a, c)


# --------------------------------------------------------------------------
# closed-form layer cases of the reference's unit tests
# --------------------------------------------------------------------------

def _uniform_layer(w13_byte, w2_byte, *, M=16, hidden=128, ispp=64, E=1, scale13=127, scale2=127,
                   a_val=1.0, top_k=1, sorted_ids=None, expert_ids=None, EM=16, out_init=0.0,
                   **kw):
    A = np.full((M, hidden), f2bf(a_val), np.uint16)
    w13 = np.full((E, 2 * ispp, hidden // 2), w13_byte, np.uint8)
    w13s = np.full((E, 2 * ispp, hidden // 32), scale13, np.uint8)
    w2 = np.full((E, hidden, ispp // 2), w2_byte, np.uint8)
    w2s = np.full((E, hidden, ispp // 32), scale2, np.uint8)
    sids = np.arange(EM, dtype=np.int32) if sorted_ids is None else sorted_ids
    eids = np.zeros(EM // 16, np.int32) if expert_ids is None else expert_ids
    out = np.full((M, hidden), out_init, np.float32)
    tws = np.ones(EM, np.float32)
    out, act = oracle.fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tws, eids, M, hidden, ispp, top_k,
                                      EM, out=out, **kw)
    return out, bf2f(act)


def test_tiny_sanity_all_ones():
    # test_moe_fused.cpp:71-120
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1))
    silu = 128.0 / (1.0 + math.exp(-128.0))
    assert np.all(np.abs(act - silu * 128) < 0.5)
    assert np.all(np.abs(out - silu * 128 * 64) / (silu * 128 * 64) < 1e-2)
    # with exact bf16 arithmetic the value is known exactly: act = bf16(16384)
    assert np.all(act == 16384.0) and np.all(out == 16384.0 * 64)


def test_bias_only():
    # test_moe_fused.cpp:125-166
    b13 = np.concatenate([np.full(64, 1.0), np.full(64, 2.0)]).astype(np.float32)[None]
    b2 = np.ones((1, 128), np.float32)
    out, act = _uniform_layer(0, 0, a_val=0.0, b13=b13, b2=b2)
    silu1 = 1.0 / (1.0 + math.exp(-1.0))
    assert np.all(np.abs(act - silu1 * 2.0) < 1e-2)
    assert np.all(np.abs(out - 1.0) < 1e-4)


def test_swiglu_clamp():
    # test_moe_fused.cpp:171-211
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1), swiglu_limit=10.0)
    want = 10.0 / (1.0 + math.exp(-10.0)) * 10.0
    assert np.all(np.abs(act - want) < 0.2)
    assert np.all(np.abs(out - want * 64) / (want * 64) < 1e-2)


def test_swiglu_clamp_is_one_sided_on_gate():
    # moe_fused.cpp:219-223: gate is clamped from above only, up on both sides
    out, act = _uniform_layer(pack_pair(-1, -1), pack_pair(1, 1), swiglu_limit=10.0)
    g = -128.0
    want = g / (1.0 + math.exp(-g)) * -10.0
    assert np.allclose(act, want, rtol=1e-2, atol=1e-30)


def test_situ_and_passthrough():
    # test_moe_fused.cpp:221-282
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1), swiglu_limit=1.0, activation=1,
                              beta=4.0, linear_beta=25.0)
    sig = 1.0 / (1.0 + math.exp(-128.0))
    want = 4.0 * math.tanh(128 / 4.0) * sig * 25.0 * math.tanh(128 / 25.0)
    assert np.all(np.abs(act - want) < 0.5)
    assert np.all(np.abs(out - want * 64) / (want * 64) < 1e-2)
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1), swiglu_limit=1.0, activation=1,
                              beta=4.0, linear_beta=0.0)
    assert np.all(np.abs(act - 4.0 * math.tanh(32.0) * sig * 128.0) < 0.5)


def test_quarter_code_and_nonfinite_codes():
    # test_moe_fused.cpp:291-367
    out, act = _uniform_layer(0x11, 0x11)
    g = 32.0
    assert np.all(np.abs(act - g / (1 + math.exp(-g)) * g) < 0.5)
    assert np.all(np.isfinite(out)) and np.all(out > 0)
    out, act = _uniform_layer(0x76, 0x22)
    assert np.all(np.isnan(act)) and np.all(np.isnan(out))


def test_subnormal_scale_underflows_to_zero():
    # test_moe_fused.cpp:369-404
    out, act = _uniform_layer(0x22, 0x22, scale13=0, scale2=0)
    assert np.all(np.abs(act) < 1e-30) and np.all(np.abs(out) < 1e-30)


def test_padding_rows_untouched_and_expert_filter():
    # test_moe_fused.cpp:406-445 and :501-533
    sids = np.full(16, 8, np.int32)
    sids[:8] = np.arange(8)
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1), M=8, sorted_ids=sids)
    assert np.all(out == 16384.0 * 64)
    assert np.all(act[8:] == 0.0) and np.all(act[:8] == 16384.0)
    out, act = _uniform_layer(pack_pair(1, 1), pack_pair(1, 1), expert_ids=np.array([-1], np.int32),
                              out_init=99.0)
    assert np.all(out == 99.0)


def test_k3_routing_top16():
    # test_moe_fused.cpp:669-736: one token fans out to 16 experts of 256
    M, hidden, ispp, top_k, E = 1, 128, 64, 16, 256
    one = pack_pair(1, 1)
    A = np.full((M, hidden), f2bf(1.0), np.uint16)
    w13 = np.full((E, 2 * ispp, hidden // 2), one, np.uint8)
    w13s = np.full((E, 2 * ispp, hidden // 32), 127, np.uint8)
    w2 = np.full((E, hidden, ispp // 2), one, np.uint8)
    w2s = np.full((E, hidden, ispp // 32), 127, np.uint8)
    ids = np.arange(16, dtype=np.int32)[None]
    sids, eids, em = oracle.moe_align_block_size(ids, 16, E)
    assert em == 256
    tws = oracle.gather_sorted_weights(np.ones(16, np.float32), sids[:em])
    assert int((tws > 0).sum()) == top_k
    out, act = oracle.fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tws, eids, M, hidden, ispp, top_k, em)
    act = bf2f(act)
    real = sids[:em] < 16
    assert np.all(act[real] == 16384.0) and np.all(act[~real] == 0.0)
    assert np.all(out == 16 * 16384.0 * 64)


def test_combine_weights_and_accumulates():
    """out accumulates (caller-zeroed) and scales by the sorted routing weight."""
    sids = np.arange(16, dtype=np.int32)
    A = np.full((16, 128), f2bf(1.0), np.uint16)
    one = pack_pair(1, 1)
    w13 = np.full((1, 128, 64), one, np.uint8); w13s = np.full((1, 128, 4), 127, np.uint8)
    w2 = np.full((1, 128, 32), one, np.uint8); w2s = np.full((1, 128, 2), 127, np.uint8)
    tws = np.linspace(0.25, 4.0, 16).astype(np.float32)
    out = np.full((16, 128), 5.0, np.float32)
    out, _ = oracle.fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tws, np.zeros(1, np.int32), 16, 128,
                                    64, 1, 16, out=out)
    assert np.array_equal(out, (5.0 + 16384.0 * 64 * tws)[:, None].astype(np.float32)
                          * np.ones((1, 128), np.float32))


# --------------------------------------------------------------------------
# alignment
# --------------------------------------------------------------------------

def align_independent(ids_flat, block_size, num_experts):
    """Written from the contract, not from the oracle's code."""
    n = len(ids_flat)
    sids, eids = [], []
    for e in range(num_experts):
        mine = [i for i, x in enumerate(ids_flat) if x == e]
        if not mine:
            continue
        pad = (-len(mine)) % block_size
        sids += mine + [n] * pad
        eids += [e] * ((len(mine) + pad) // block_size)
    return np.array(sids, np.int32), np.array(eids, np.int32), len(sids)


def test_align_basic_example():
    # test_moe_fused.cpp:538-581 and docs/kernels/moe_fused.md:317-331
    ids = np.array([[0] * 4, [0, 1, 1, 1], [1] * 4, [1] * 4, [2] * 4, [2] * 4, [2] * 4, [2] * 4],
                   np.int32)
    sids, eids, em = oracle.moe_align_block_size(ids, 16, 4)
    assert em == 48 and list(eids[:3]) == [0, 1, 2]
    assert list(sids[:5]) == [0, 1, 2, 3, 4] and np.all(sids[5:16] == 32)
    assert list(sids[32:48]) == list(range(16, 32))


def test_align_padding_sentinels_exact():
    # test_moe_align_oracle.cpp:87-105
    ids = np.array([[-1, -1], [1, -1], [1, -1]], np.int32)
    sids, eids, em = oracle.moe_align_block_size(ids, 16, 4, fill=(-777, -888))
    assert em == 16 and eids[0] == 1 and sids[0] == 2 and sids[1] == 4
    assert np.all(sids[2:16] == 6) and np.all(sids[16:] == -777) and np.all(eids[1:] == -888)


def test_align_garbage_ids_skipped():
    # test_moe_align_oracle.cpp:111-133
    ids = np.array([[0, 99, -3, 1, 4, 1, 2, -1]], np.int32)
    sids, eids, em = oracle.moe_align_block_size(ids, 16, 4)
    assert em == 48 and list(eids[:3]) == [0, 1, 2]
    assert sids[0] == 0 and sids[16] == 3 and sids[17] == 5 and sids[32] == 6
    assert np.all((sids[:em] >= 0) & (sids[:em] <= 8))


@pytest.mark.parametrize("M,k,E,bs", [(17, 2, 8, 64), (64, 8, 256, 16), (5, 16, 256, 64),
                                      (33, 1, 7, 32), (1, 4, 32, 16), (100, 6, 64, 16)])
def test_align_matches_independent_reference(M, k, E, bs):
    # test_moe_align_oracle.cpp:139-171
    rng = np.random.default_rng(M * 131 + E)
    ids = rng.integers(-2, E + 2, (M, k)).astype(np.int32)
    sids, eids, em = oracle.moe_align_block_size(ids, bs, E)
    rs, re_, rem = align_independent(list(ids.ravel()), bs, E)
    assert em == rem and np.array_equal(sids[:em], rs) and np.array_equal(eids[:em // bs], re_)
    if oracle.have_ref():
        s2, e2, em2 = oracle.moe_align_block_size(ids, bs, E, use_ref=True)
        assert em2 == em and np.array_equal(s2, sids) and np.array_equal(e2, eids)


def test_align_m0_returns_zero_rows():
    # test_moe_align_oracle.cpp:237-244
    _, _, em = oracle.moe_align_block_size(np.zeros((0, 2), np.int32), 16, 4)
    assert em == 0


def test_align_with_map_semantics():
    """Serving semantics: remap, min one block, all max_EM entries written."""
    ids = np.array([3, 0, 2, 3, 1, 7, -1], np.int32)
    emap = np.array([1, -1, 0, 1], np.int32)           # experts 0,3 -> local 1; 2 -> local 0
    s, e, em = oracle.moe_align_block_size_with_map(ids, 4, 4, emap, local_n=2, max_EM=16)
    assert em == 8 and list(e) == [0, 1, -1, -1]
    assert list(s) == [2, 7, 7, 7, 0, 1, 3, 7] + [7] * 8
    s, e, em = oracle.moe_align_block_size_with_map(np.array([9, -4], np.int32), 4, 16, None,
                                                    max_EM=32)
    assert em == 16 and np.all(s == 2) and np.all(e == -1)


def test_em_bound_upper_bounds_oracle():
    # test_moe_align_oracle.cpp:180-232
    for (M, k, E, bs) in [(1, 8, 32, 16), (8, 8, 32, 16), (50, 8, 32, 64), (32, 16, 896, 64),
                          (1, 16, 256, 16), (4, 8, 256, 16)]:
        N = M * k
        bound = oracle.align_em_bound(M, k, E, bs)
        assert bound >= N and bound % bs == 0
        rng = np.random.default_rng(N * 31 + E)
        for kind in ("uniform", "hot", "power"):
            if kind == "uniform":
                ids = rng.integers(0, E, N)
            elif kind == "hot":
                ids = np.where(rng.random(N) < 0.9, 0, rng.integers(0, E, N))
            else:
                ids = np.minimum(rng.geometric(0.5, N) - 1, E - 1)
            _, _, em = oracle.moe_align_block_size(ids.reshape(M, k).astype(np.int32), bs, E)
            assert bound >= em
    assert oracle.align_em_bound(0, 4, 8, 16) == 16
    assert oracle.align_max_em(8, 4, 16, 4) == (2 + 4) * 16


# --------------------------------------------------------------------------
# golden fixtures (outputs of the reference build) and the live reference
# --------------------------------------------------------------------------

def _load_case(name):
    d = np.load(GOLDEN / f"{name}.npz")
    cfg = synth.CONFIGS.get(str(d["cfg"])) or synth.MoEConfig("c9", 128, 64, 4, 2, (5,), "uniform")
    T, seed = int(d["T"]), int(d["seed"])
    w = synth.make_weights(cfg.E, cfg.H, cfg.I, seed).numpy()
    A = synth.make_activations(T, cfg.H, seed)
    chk = [int(A.astype(np.uint64).sum()), int(w[0].astype(np.uint64).sum()),
           int(w[2].astype(np.uint64).sum())]
    assert chk == list(d["checksum_inputs"]), "input generator no longer reproduces the fixture inputs"
    kw = json.loads(str(d["kw"]))
    b13 = b2 = None
    if bool(d["bias"]):
        b13 = synth.rand_normal((cfg.E, 2 * cfg.I), seed, 21).astype(np.float32)
        b2 = synth.rand_normal((cfg.E, cfg.H), seed, 22).astype(np.float32)
    return d, cfg, T, seed, w, A, kw, b13, b2


@pytest.mark.parametrize("name", ["c0_T16_swiglu", "c0_T16_swiglu_limit_bias", "c0_T16_situ_bias",
                                  "small_T5"])
def test_layer_matches_reference_fixture_bitwise(name):
    d, cfg, T, seed, w, A, kw, b13, b2 = _load_case(name)
    ids = d["topk_ids"]
    sids, eids, em = oracle.moe_align_block_size(ids, 16, cfg.E)
    assert em == int(d["EM"])
    assert np.array_equal(sids[:em], d["sorted_ids"]) and np.array_equal(eids[:em // 16], d["expert_ids"])
    tws = oracle.gather_sorted_weights(d["topk_w"], sids[:em])
    for threads in (1, 4):
        oracle.set_threads(threads)
        out, act = oracle.fused_moe_mxfp4(A, *w, sids, tws, eids, T, cfg.H, cfg.I, cfg.top_k, em,
                                          b13=b13, b2=b2, **kw)
        assert np.array_equal(out.view(np.uint32), d["out"].view(np.uint32))
        assert np.array_equal(act[:em], d["act"])
    oracle.set_threads(1)


def test_align_matches_reference_fixture():
    d = np.load(GOLDEN / "align_cases.npz")
    for i in range(int(d["n"])):
        M, k, E, bs, em_ref = (int(x) for x in d[f"meta{i}"])
        sids, eids, em = oracle.moe_align_block_size(d[f"ids{i}"], bs, E)
        assert em == em_ref
        assert np.array_equal(sids[:em], d[f"sids{i}"]) and np.array_equal(eids[:em // bs], d[f"eids{i}"])


@pytest.mark.skipif(not oracle.have_ref(), reason="reference build oracle/_ref not present")
def test_stage_functions_match_live_reference():
    """Stage split with a K slice (k_base > 0), padding rows and a filtered block."""
    rng = np.random.default_rng(3)
    M, H, I, E, k = 9, 192, 128, 5, 3
    w = synth.make_weights(E, H, I, 99).numpy()
    A = synth.make_activations(M, H, 99)
    ids = rng.integers(0, E, (M, k)).astype(np.int32)
    sids, eids, em = oracle.moe_align_block_size(ids, 16, E)
    sids, eids = sids[:em].copy(), eids[:em // 16].copy()
    eids[1] = -1
    for (kb, kd) in ((0, H), (64, 128), (128, 64)):
        w13 = np.ascontiguousarray(w[0][:, :, kb // 2:(kb + kd) // 2])
        w13s = np.ascontiguousarray(w[1][:, :, kb // 32:(kb + kd) // 32])
        a = oracle.moe_gateup(A, w13, w13s, sids, eids, M, H, kb, kd, I, k, em, fill=7.0)
        b = oracle.moe_gateup(A, w13, w13s, sids, eids, M, H, kb, kd, I, k, em, fill=7.0, use_ref=True)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    gu = oracle.moe_gateup(A, w[0], w[1], sids, eids, M, H, 0, H, I, k, em)
    b13 = rng.normal(size=(E, 2 * I)).astype(np.float32)
    for kw in (dict(), dict(swiglu_limit=3.0), dict(activation=1, beta=2.0, linear_beta=5.0),
               dict(activation=1, linear_beta=0.0)):
        a = oracle.moe_act_epilogue(gu, b13, sids, eids, M, k, em, I, **kw)
        b = oracle.moe_act_epilogue(gu, b13, sids, eids, M, k, em, I, use_ref=True, **kw)
        assert np.array_equal(a, b)
    act = oracle.moe_act_epilogue(gu, None, sids, eids, M, k, em, I)
    for (kb, kd) in ((0, I), (64, 64)):
        w2 = np.ascontiguousarray(w[2][:, :, kb // 2:(kb + kd) // 2])
        w2s = np.ascontiguousarray(w[3][:, :, kb // 32:(kb + kd) // 32])
        a = oracle.moe_down(act, w2, w2s, sids, eids, M, I, kb, kd, H, k, em, fill=3.0)
        b = oracle.moe_down(act, w2, w2s, sids, eids, M, I, kb, kd, H, k, em, fill=3.0, use_ref=True)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    partial = oracle.moe_down(act, w[2], w[3], sids, eids, M, I, 0, I, H, k, em)
    tws = rng.random(em).astype(np.float32)
    b2 = rng.normal(size=(E, H)).astype(np.float32)
    a = oracle.moe_combine(partial, b2, tws, sids, eids, M, H, k, em)
    b = oracle.moe_combine(partial, b2, tws, sids, eids, M, H, k, em, use_ref=True)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.skipif(not oracle.have_ref(), reason="reference build oracle/_ref not present")
@pytest.mark.parametrize("T,H,I,E,k,seed", [(3, 64, 64, 2, 1, 1), (40, 256, 192, 6, 3, 2),
                                            (70, 128, 320, 16, 4, 3)])
def test_fused_matches_live_reference(T, H, I, E, k, seed):
    w = synth.make_weights(E, H, I, seed, scale_lo=107, scale_hi=147).numpy()
    A = synth.make_activations(T, H, seed)
    lg = synth.make_logits("uniform", T, E, seed)
    oracle.set_threads(3)
    a = oracle.moe_layer(A, lg, *w, k)
    b = oracle.moe_layer(A, lg, *w, k, use_ref=True)
    oracle.set_threads(1)
    assert a["EM"] == b["EM"]
    assert np.array_equal(a["out"].view(np.uint32), b["out"].view(np.uint32))
    assert np.array_equal(a["act"], b["act"])


# --------------------------------------------------------------------------
# router (no reference CPU code: closed forms, brute force, torch as a library)
# --------------------------------------------------------------------------

def test_route_exp_accuracy():
    xs = np.concatenate([-np.logspace(-6, 1.9, 400), [0.0, -79.9, -80.0, -81.0, -1e30]])
    for x in xs:
        got = oracle.route_exp(float(np.float32(x)))
        want = math.exp(float(np.float32(x))) if x > -80.0 else 0.0
        assert got == pytest.approx(want, rel=3e-7, abs=0.0)
    assert oracle.route_exp(0.0) == 1.0


def test_router_closed_forms():
    # equal logits: uniform probabilities, ties to the lowest index, weights 1/k
    ids, w = oracle.route_topk(np.zeros((2, 8), np.float32), 3, True)
    assert ids.tolist() == [[0, 1, 2]] * 2 and np.allclose(w, 1 / 3)
    # two-expert softmax = sigmoid of the difference
    lg = np.array([[0.0, 1.0], [2.0, -1.0]], np.float32)
    ids, w = oracle.route_topk(lg, 2, False)
    assert ids.tolist() == [[1, 0], [0, 1]]
    assert w[0, 0] == pytest.approx(1 / (1 + math.exp(-1.0)), rel=1e-6)
    assert w[1, 1] == pytest.approx(1 / (1 + math.exp(3.0)), rel=1e-6)
    # renormalised weights sum to one; a far-away expert underflows to exactly 0
    lg = np.array([[0.0, -100.0, -0.5, -200.0]], np.float32)
    ids, w = oracle.route_topk(lg, 4, True)
    assert ids.tolist() == [[0, 2, 1, 3]] and w[0, 2] == 0.0 and w[0, 3] == 0.0
    assert float(w.sum()) == pytest.approx(1.0, rel=1e-6)


def test_router_against_torch_library():
    import torch
    for (T, E, k, seed) in [(64, 32, 4, 1), (128, 128, 4, 2), (64, 256, 8, 3), (16, 384, 16, 4)]:
        lg = synth.make_logits("uniform", T, E, seed)
        ids, w = oracle.route_topk(lg, k, True)
        p = torch.softmax(torch.from_numpy(lg).double(), dim=-1)
        tv, ti = torch.topk(p, k, dim=-1)
        # indices must agree wherever the k-th/(k+1)-th and neighbouring gaps are clear
        srt = torch.sort(p, dim=-1, descending=True).values[:, :k + 1]
        clear = ((srt[:, :-1] - srt[:, 1:]) / srt[:, :-1] > 1e-5).all(dim=-1).numpy()
        assert clear.mean() > 0.9
        assert np.array_equal(ids[clear], ti.numpy()[clear].astype(np.int32))
        wn = (tv / tv.sum(dim=-1, keepdim=True)).numpy()
        assert np.allclose(w[clear], wn[clear], rtol=2e-6, atol=0)
        # invariants on every row
        assert all(len(set(r)) == k for r in ids.tolist())
        assert np.allclose(w.sum(axis=1), 1.0, rtol=1e-6)
        assert np.all(np.diff(w, axis=1) <= 0)


def test_router_brute_force_ties():
    rng = np.random.default_rng(0)
    for _ in range(200):
        E, k = int(rng.integers(2, 9)), 2
        lg = rng.integers(-2, 3, (1, E)).astype(np.float32)   # many exact ties
        ids, _ = oracle.route_topk(lg, k, True)
        order = sorted(range(E), key=lambda e: (-lg[0, e], e))
        assert ids[0].tolist() == order[:k]


# --------------------------------------------------------------------------
# the reference's CPU C ABI as served by the oracle library
# --------------------------------------------------------------------------

def test_cpu_abi_status_codes_and_null_guards():
    # tests/capi/test_capi.cpp:1484-1647
    import ctypes
    lib = oracle.lib()
    lib.vk_last_error.restype = ctypes.c_char_p
    out_em = ctypes.c_int32(-1)
    ids = (ctypes.c_int32 * 4)(0, 1, 0, 1)
    s = (ctypes.c_int32 * 64)()
    e = (ctypes.c_int32 * 4)()
    assert lib.vk_moe_align_block_size(ids, 2, 2, 16, 2, s, e, ctypes.byref(out_em)) == 0
    assert out_em.value == 32
    assert lib.vk_moe_align_block_size(ids, 2, 2, 0, 2, s, e, ctypes.byref(out_em)) == 1
    assert b"block_size" in lib.vk_last_error() and lib.vk_last_error_code() == 1
    assert lib.vk_moe_align_block_size(None, 2, 2, 16, 2, s, e, ctypes.byref(out_em)) == 1
    assert lib.vk_moe_align_block_size(ids, 2, 2, 16, 2, s, e, None) == 1
    assert lib.vk_moe_align_block_size(None, 0, 2, 16, 2, s, e, ctypes.byref(out_em)) == 0
    assert out_em.value == 0
    lib.vk_moe_align_block_size_max_em.restype = ctypes.c_size_t
    assert lib.vk_moe_align_block_size_max_em(8, 4, 16, 4) == 96
    assert lib.vk_moe_align_block_size_max_em(8, 4, 0, 4) == 0
    f = ctypes.c_float
    args_tail = (16, 128, 64, 1, 16, 32, f(0.0), 0, f(4.0), f(25.0), None, None)
    assert lib.vk_fused_moe_mxfp4(*([None] * 10), *args_tail) == 1          # null buffers
    assert lib.vk_fused_moe_mxfp4(*([None] * 10), 0, 128, 64, 1, 0, 32, f(0.0), 0, f(4.0), f(25.0),
                                  None, None) == 0                          # M = 0 is a no-op
