"""GPU parity of the prefill-sized path on prepacked weights (FP4 x FP6 scaled MFMA),
through the C ABI.

Bit-exact: the prepacked layout, the split rows (against the oracle's model of the
activation operands), and the weight values the matrix cores multiply by (one-hot
activation rows through the second stage, every kernel family).
Layer output: against the oracle within the contract's tolerance, and against the
oracle run with the same activation representation (`oracle.set_act_model`) within a
ten times tighter one, which isolates the GPU's accumulation from the representation.
"""
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
                      edge_tokens, error_metrics, to_dev)

pytestmark = pytest.mark.gpu

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

# GPU against the oracle that multiplies the same activation representation: what is
# left is the order of the fp32 sums and bf16 roundings of act that fall the other way
MODEL_REL_L2_TOL = 5e-4
MODEL_MAX_ABS_TOL = 5e-3


# ---- the prepacked layout ---------------------------------------------------------

def _prepack_reference(w, ws, stage):
    """numpy restatement of the packed layout documented in include/vkernels_hip.h: a flagged
    unit holds the codes and scale bytes as they are, any other the codes on the OCP points
    and the scale bytes less one."""
    E, rows, kb = w.shape
    K = kb * 2
    ncols = rows // 2 if stage == 0 else rows
    units = ncols // 64 if stage == 0 else (ncols + 127) // 128
    ksteps = (K + 127) // 128
    out = np.zeros((E, units, ksteps, 8704), dtype=np.uint8)
    flags = np.zeros((E, units), dtype=np.uint8)
    lo, hi = w & 15, w >> 4
    remap = lambda c: c + np.where((c & 6) != 0, 2, 0).astype(np.uint8)
    nonfinite = ((lo & 6) == 6) | ((hi & 6) == 6)
    bad_row = nonfinite.any(axis=2) | (ws < 64).any(axis=2) | (ws > 190).any(axis=2)
    for e in range(E):
        for u in range(units):
            rows_u = [(t >> 1) * ncols + u * 64 + (t & 1) * 32 + n if stage == 0 else u * 128 + t * 32 + n
                      for t in range(4) for n in range(32)]
            raw = any(r < rows and bad_row[e, r] for r in rows_u)
            for t in range(4):
                for n in range(32):
                    row = (t >> 1) * ncols + u * 64 + (t & 1) * 32 + n if stage == 0 else u * 128 + t * 32 + n
                    if row >= rows:
                        for ks in range(ksteps):
                            out[e, u, ks, 8192:].reshape(64, 2, 4)[[n, n + 32], :, t] = 127
                        continue
                    if nonfinite[e, row].any() or (ws[e, row] < 64).any() or (ws[e, row] > 190).any():
                        flags[e, u] = 1
                    for g in range(ksteps * 4):
                        ks, half, hh = g // 4, (g // 2) % 2, g % 2
                        lane = n + 32 * hh
                        sc_view = out[e, u, ks, 8192:].reshape(64, 2, 4)
                        if g * 32 >= K:
                            sc_view[lane, half, t] = 127
                            continue
                        piece = w[e, row, g * 16:(g + 1) * 16]
                        packed = piece if raw else remap(piece & 15) | (remap(piece >> 4) << 4)
                        off = ((half * 4 + t) * 64 + lane) * 16
                        out[e, u, ks, off:off + 16] = packed
                        sc_view[lane, half, t] = int(ws[e, row, g]) if raw else (int(ws[e, row, g]) - 1) & 0xFF
    return out, flags


@pytest.mark.parametrize("stage,rows,K", [(0, 256, 192), (1, 192, 128), (1, 128, 320)])
def test_prepack_layout_bitwise(hip_lib, stage, rows, K):
    size_fn, pack_fn, _ = ve.resolve_prepack_fns(hip_lib)
    E = 3
    rng = np.random.default_rng(stage * 100 + rows)
    fin = np.array(synth.FINITE_CODES, dtype=np.uint8)
    w = (fin[rng.integers(0, 12, (E, rows, K // 2))] | (fin[rng.integers(0, 12, (E, rows, K // 2))] << 4)).astype(np.uint8)
    ws = rng.integers(64, 191, (E, rows, K // 32)).astype(np.uint8)
    w[1, 7, 3] = 0x6E           # an inf code: its unit is flagged
    ws[2, rows - 1, 0] = 63     # a scale byte below the range: its unit is flagged
    ws[0, 40, 1] = 191          # above the range
    n = int(size_fn(E, rows, K, stage))
    buf = torch.zeros(n, dtype=torch.uint8, device=dev())
    d_w, d_ws = to_dev(w), to_dev(ws)
    st = pack_fn(d_w.data_ptr(), d_ws.data_ptr(), E, rows, K, stage, buf.data_ptr(), n, None)
    assert st == 0, ve.last_error(hip_lib)
    torch.cuda.synchronize()
    ref, flags = _prepack_reference(w, ws, stage)
    got = buf.cpu().numpy()
    body = ref.size
    # byte for byte, the flagged units (raw codes and scale bytes for the exact paths) included
    assert np.array_equal(got[:body], ref.ravel())
    f_off = (body + 255) // 256 * 256
    assert np.array_equal(got[f_off:f_off + flags.size], flags.ravel())
    assert flags.sum() == 3


# ---- the split rows ------------------------------------------------------------------

def _decode_fp6(codes24):
    """[..., 24] bytes -> [..., 32] floats (E2M3, code i at bit 6 i)."""
    b = codes24.astype(np.uint64)
    bits = np.zeros(codes24.shape[:-1] + (3,), dtype=np.uint64)
    for i in range(3):
        for j in range(8):
            bits[..., i] |= b[..., 8 * i + j] << np.uint64(8 * j)
    vals = np.zeros(codes24.shape[:-1] + (32,), dtype=np.float64)
    for i in range(32):
        bit = 6 * i
        word, sh = bit // 64, bit % 64
        c = (bits[..., word] >> np.uint64(sh))
        if sh > 58:
            c |= bits[..., word + 1] << np.uint64(64 - sh)
        c = (c & np.uint64(63)).astype(np.int64)
        e, m = (c >> 3) & 3, c & 7
        v = np.where(e == 0, m / 8.0, np.ldexp(1.0 + m / 8.0, e - 1))
        vals[..., i] = np.where(c & 32, -v, v)
    return vals


@pytest.mark.parametrize("terms", [2, 3])
def test_split_rows_match_the_oracle_model(hip_lib, terms):
    fn = hip_lib.vk_hip_split_rows_fp6
    fn.restype = _I
    fn.argtypes = [_P, _I, _I, _I, _P, _P, _P]
    rows, K = 24, 2880
    kp = (K + 127) // 128 * 128
    x = synth.make_activations(rows, K, 77 + terms)
    xf = synth.bf16_bits_to_f32(x)
    x[1] = synth.f32_to_bf16_bits(xf[1] * np.float32(2.0 ** 40))
    x[2] = synth.f32_to_bf16_bits(xf[2] * np.float32(2.0 ** -40))
    x[3, 64:96] = 0                      # a block of zeros
    x[4, 100] = 0x7F80                   # inf: the row is flagged
    x[5, 7] = 0x7FC0                     # NaN
    x[6] = synth.f32_to_bf16_bits(xf[6] * np.float32(2.0 ** 90))    # scale byte above 190
    x[7] = synth.f32_to_bf16_bits(xf[7] * np.float32(2.0 ** -70))   # below the range
    x[8, 5] = 0x40FF                     # 7.96875: saturates the first term
    out = torch.zeros(rows * terms * kp, dtype=torch.uint8, device=dev())
    flags = torch.full((rows,), 9, dtype=torch.uint8, device=dev())
    d_x = to_dev(x)
    st = fn(d_x.data_ptr(), rows, K, terms, out.data_ptr(), flags.data_ptr(), None)
    assert st == 0, ve.last_error(hip_lib)
    torch.cuda.synchronize()
    fl = flags.cpu().numpy()
    assert list(np.nonzero(fl)[0]) == [4, 5, 6, 7], fl
    blocks = out.cpu().numpy().reshape(rows, terms, kp // 32, 32)
    vals = _decode_fp6(blocks[..., :24])                        # [rows, terms, nblk, 32]
    scale = np.ldexp(1.0, blocks[..., 24].astype(np.int64) - 127)
    assert not blocks[..., 25:].any()
    total = (vals * scale[..., None]).sum(axis=1)                # [rows, nblk, 32]
    for r in range(rows):
        if fl[r]:
            continue
        for b in range(kp // 32):
            if b * 32 >= K:
                assert not total[r, b].any()
                continue
            model = oracle.act_model_block32(x[r, b * 32:(b + 1) * 32], terms).astype(np.float64)
            assert np.array_equal(total[r, b], model), (r, b)
    # three terms resolve 2^-13 of the block's largest: exact but for the elements below
    # 2^-5 of it (a few percent of a normal block), which are off by at most 2^-14 of it
    if terms == 3:
        exact = synth.bf16_bits_to_f32(x[9:]).astype(np.float64).reshape(rows - 9, K // 32, 32)
        err = np.abs(total[9:, :K // 32] - exact)
        big = np.abs(exact).max(axis=2, keepdims=True)
        assert (err <= 2.0 ** -14 * big).all()
        assert not err[np.abs(exact) >= 2.0 ** -5 * big].any()
        assert np.count_nonzero(err) < 0.03 * err.size


# ---- the weight values the kernels multiply by ---------------------------------------

def _down_ex(lib):
    fn = lib.vk_hip_moe_down_mxfp4_ex
    fn.restype = None
    fn.argtypes = [_P] * 5 + [_I] * 4 + [_P, _P, _I, _P, _I, _P, ctypes.c_size_t, ctypes.c_uint, _P, _I, _P]
    return fn


@pytest.mark.parametrize("path", ["packed", "packed3", "packed2", "workspace", "plain", "resident",
                                  "packed_alone", "resident_packed_alone"])
def test_onehot_rows_read_back_the_dequantised_weights(hip_lib, path):
    """act rows with a single 1.0 at column k, routing weight 1: out[t, :] is column k of
    the expert's dequantised W2, so every value the GEMM multiplies by is compared with the
    oracle bit for bit.  Expert 0: the 12 finite codes with scale bytes 64, 65, 127, 189,
    190 (the scaled-MFMA path); expert 1: all 16 codes and scale bytes 0, 1, 63, 191, 200,
    255 (flagged: the exact path).  The paths "..._alone" pass the prepacked form and no raw
    tensors: the flagged units' raw codes and scale bytes are then read from it."""
    E, H = 2, 192
    alone = path.endswith("_alone")
    I = 256 if path.startswith("resident") else 576
    M = E * I
    rng = np.random.default_rng(11)
    fin = np.array(synth.FINITE_CODES, dtype=np.uint8)
    w2 = np.zeros((E, H, I // 2), dtype=np.uint8)
    w2[0] = fin[rng.integers(0, 12, (H, I // 2))] | (fin[rng.integers(0, 12, (H, I // 2))] << 4)
    w2[1] = rng.integers(0, 256, (H, I // 2)).astype(np.uint8)
    keep = np.ones(H, dtype=bool)
    keep[[5, 77]] = False                                          # rows that keep their inf/NaN codes
    lo, hi = w2[1] & 15, w2[1] >> 4
    lo[keep] = fin[lo[keep] % 12]
    hi[keep] = fin[hi[keep] % 12]
    w2[1] = lo | (hi << 4)
    w2s = np.zeros((E, H, I // 32), dtype=np.uint8)
    w2s[0] = np.array([64, 65, 127, 189, 190], dtype=np.uint8)[rng.integers(0, 5, (H, I // 32))]
    w2s[1] = np.array([0, 1, 63, 191, 200, 255], dtype=np.uint8)[rng.integers(0, 6, (H, I // 32))]
    ids = (np.arange(M) // I).astype(np.int32).reshape(M, 1)
    fe = ve.FusedExperts(to_dev(np.zeros((E, 2 * I, H // 2), np.uint8)), to_dev(np.zeros((E, 2 * I, H // 32), np.uint8)),
                         to_dev(w2), to_dev(w2s), scratch=ve.CaptureSafeScratch(),
                         prepack=path.startswith("packed") or alone, keep_raw=not alone)
    bs = 16 if path.startswith("resident") else 128
    sids, eids, out_em, max_em = fe.align(to_dev(ids), bs)
    torch.cuda.synchronize()
    s_np = sids.cpu().numpy()
    act = np.zeros((max_em, I), dtype=np.uint16)
    real = np.nonzero(s_np < M)[0]
    act[real, s_np[real] % I] = 0x3F80                              # 1.0
    d_act = to_dev(act)
    tw = torch.ones((M, 1), dtype=torch.float32, device=dev())
    out = torch.full((M, H), float("nan"), dtype=torch.float32, device=dev())
    ws, need = None, 0
    if path != "plain" and not path.startswith("resident"):
        need = int(fe.ws_bytes_fn(M, H, I, 1, max_em))
        ws = torch.empty(need, dtype=torch.uint8, device=dev())
    flags = ve.MOE_OVERWRITE_OUT | (ve.MOE_SPLIT2 if path == "packed2" else ve.MOE_SPLIT3 if path == "packed3" else 0)
    hip_lib.vk_set_last_error(0, b"")
    _down_ex(hip_lib)(d_act.data_ptr(), None if alone else fe.w2.data_ptr(),
                      None if alone else fe.w2_scale.data_ptr(), tw.data_ptr(),
                      out.data_ptr(), M, H, I, 1, sids.data_ptr(), eids.data_ptr(), max_em, None, bs,
                      None if ws is None else ws.data_ptr(), need, flags,
                      None if fe.w2_packed is None else fe.w2_packed.data_ptr(), E, None)
    torch.cuda.synchronize()
    assert hip_lib.vk_last_error_code() == 0, ve.last_error(hip_lib)
    got = out.cpu().numpy()
    # expected: the oracle's second stage on the same act
    eids16 = np.repeat(eids.cpu().numpy(), bs // 16).astype(np.int32)
    partial = oracle.moe_down(act, w2, w2s, s_np, eids16, M, I, 0, I, H, 1, max_em)
    tws = oracle.gather_sorted_weights(tw.cpu().numpy(), s_np)
    exp = oracle.moe_combine(partial, None, tws, s_np, eids16, M, H, 1, max_em)
    same = (got == exp) | (np.isnan(got) & np.isnan(exp))
    assert same.all(), f"{path}: {np.count_nonzero(~same)} values differ, first at {np.argwhere(~same)[:5]}"
    # and the expectation is the dequantisation table itself for the finite expert
    table = synth.bf16_bits_to_f32(oracle.dequant_weight_tile(w2[0], w2s[0], H, I))   # [I, H]
    assert np.array_equal(exp[:I], table)
    assert np.isnan(exp[I:, 5]).all() and np.isfinite(exp[I:, 6]).all()


def _bf16_order(bits):
    """bf16 bit patterns -> integers that order like the values, +0 and -0 both 0."""
    b = bits.astype(np.int64)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)


@pytest.mark.parametrize("path", ["packed", "packed3", "packed2", "workspace", "plain", "resident",
                                  "packed_alone", "resident_packed_alone"])
def test_onehot_rows_through_the_first_stage(hip_lib, path):
    """A rows with a single 1.0 at column k: the gate and up sums of sorted row r are single
    exact products, W13[e, c, k] and W13[e, I + c, k], so act[r, c] = bf16(silu(g) u) pins
    the values the first stage multiplies by (its prepack row map and its template
    instantiations differ from the second stage's).  Expert 0: the 12 finite codes; gate
    rows take scale bytes 64, 65, 127, 189, 190 and the up row of the same column the
    mirrored byte (254 - s), so every product is of order one: a tiny g gives g / 2 * u and
    a huge positive one g * u exactly, in the oracle and in the kernels' hardware
    exponential and reciprocal alike.  Expert 1: all 16 codes in two rows, scale bytes 0,
    1, 63, 191, 200, 255 (flagged units: the exact path).  act must be within one bf16 unit
    in the last place of the oracle's everywhere, and bit-equal in at least 99 % of the
    values."""
    E, I = 2, 192
    alone = path.endswith("_alone")
    H = 256 if path.startswith("resident") else 576
    M = E * H
    rng = np.random.default_rng(23)
    fin = np.array(synth.FINITE_CODES, dtype=np.uint8)
    w13 = np.zeros((E, 2 * I, H // 2), dtype=np.uint8)
    w13[0] = fin[rng.integers(0, 12, (2 * I, H // 2))] | (fin[rng.integers(0, 12, (2 * I, H // 2))] << 4)
    w13[1] = rng.integers(0, 256, (2 * I, H // 2)).astype(np.uint8)
    keep = np.ones(2 * I, dtype=bool)
    keep[[5, I + 70]] = False                                       # rows that keep their inf/NaN codes
    lo, hi = w13[1] & 15, w13[1] >> 4
    lo[keep] = fin[lo[keep] % 12]
    hi[keep] = fin[hi[keep] % 12]
    w13[1] = lo | (hi << 4)
    w13s = np.zeros((E, 2 * I, H // 32), dtype=np.uint8)
    w13s[0, :I] = np.array([64, 65, 127, 189, 190], dtype=np.uint8)[rng.integers(0, 5, (I, H // 32))]
    w13s[0, I:] = 254 - w13s[0, :I]
    w13s[1] = np.array([0, 1, 63, 191, 200, 255], dtype=np.uint8)[rng.integers(0, 6, (2 * I, H // 32))]
    w2 = (fin[rng.integers(0, 12, (E, H, I // 2))] | (fin[rng.integers(0, 12, (E, H, I // 2))] << 4)).astype(np.uint8)
    w2s = np.full((E, H, I // 32), 127, dtype=np.uint8)
    ids = (np.arange(M) // H).astype(np.int32).reshape(M, 1)
    A = np.zeros((M, H), dtype=np.uint16)
    A[np.arange(M), np.arange(M) % H] = 0x3F80                        # 1.0
    kw = dict(prepack=path.startswith("packed") or alone, keep_raw=not alone)
    if path in ("packed2", "packed3"):
        kw["split_terms"] = int(path[-1])
    fe = ve.FusedExperts(to_dev(w13), to_dev(w13s), to_dev(w2), to_dev(w2s), scratch=ve.CaptureSafeScratch(), **kw)
    fe.use_workspace = path not in ("plain", "resident")
    bs = 16 if path.startswith("resident") else 128
    d_ids = to_dev(ids)
    sids, eids, out_em, max_em = fe.align(d_ids, bs)
    fe.apply(to_dev(A, torch.bfloat16), d_ids, None, block_size=bs)
    torch.cuda.synchronize()
    act = fe.scratch.get(("act", I), max_em * I, dtype=torch.bfloat16, device=dev())
    got = act.view(torch.int16).cpu().numpy().view(np.uint16).reshape(max_em, I)
    s_np = sids.cpu().numpy()
    # expected: the oracle's first stage on the same rows, in the same sorted order
    eids16 = np.repeat(eids.cpu().numpy(), bs // 16).astype(np.int32)
    gate_up = oracle.moe_gateup(A, w13, w13s, s_np, eids16, M, H, 0, H, I, 1, max_em)
    exp = oracle.moe_act_epilogue(gate_up, None, s_np, eids16, M, 1, max_em, I)
    real = np.nonzero(s_np < M)[0]
    first = real[s_np[real] < H]                                     # expert 0's rows: the scaled-MFMA path
    # ... where the expectation is the products themselves for the tiny and the huge gates
    g = synth.bf16_bits_to_f32(oracle.dequant_weight_tile(w13[0], w13s[0], 2 * I, H)).astype(np.float64)  # [H, 2I]
    k_of = s_np[first] % H
    gg, uu = g[k_of, :I], g[k_of, I:]
    gsc = np.repeat(w13s[0, :I].T, 32, axis=0)[k_of]                 # the gate's scale byte per (row, column)
    want = np.where(gsc <= 65, gg / 2 * uu, np.where(gg > 0, gg * uu, 0.0))
    closed = gsc != 127
    assert np.array_equal(synth.bf16_bits_to_f32(exp[first])[closed].astype(np.float64), want[closed])
    for name, rows in (("scaled MFMA path", first), ("exact path", real[s_np[real] >= H])):
        a, b = got[rows], exp[rows]
        nan_a, nan_b = (a & 0x7FFF) > 0x7F80, (b & 0x7FFF) > 0x7F80
        assert np.array_equal(nan_a, nan_b), f"{path}, {name}: NaN patterns differ"
        ok = ~nan_a
        dist = np.abs(_bf16_order(a) - _bf16_order(b))[ok]
        equal = np.mean(dist == 0)
        print(f"{path}, {name}: {rows.size} rows, bit-equal {equal:.5f}, worst distance {dist.max()} ulp")
        assert dist.max() <= 1, f"{path}, {name}: act is {dist.max()} bf16 ulps from the oracle's"
        assert equal >= 0.99


def _run_layer_rows(cfg, w, A_bits, logits, **kw):
    fe = ve.FusedExperts(w.w13, w.w13_scale, w.w2, w.w2_scale, scratch=ve.CaptureSafeScratch(), **kw)
    A = to_dev(A_bits, torch.bfloat16)
    ids, tw = fe.route(to_dev(logits), cfg.top_k, True)
    out = fe.apply(A, ids, tw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("name,T", [("c2", 4096), ("c3", 16384)])
def test_all_rows_agree_between_the_two_kernel_families(name, T):
    """Full size, every token: the prepacked call (FP4-rate kernels, three FP6 terms in both
    stages) against the raw-weight call with a workspace (FP8-rate kernels, exact two-term
    split) on the same inputs.  Two kernel families with different tilings, layouts and
    row maps: a localised error of either (a tile, a window edge, an expert's last rows)
    shows as a row that disagrees, which the oracle's sample of rows may miss.  The
    sampled rows' own distance to the oracle is measured in the tests above; here every
    row must stay inside the same bound."""
    cfg = synth.CONFIGS[name]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 2000 if name == "c2" else 3000)
    a = _run_layer_rows(cfg, w, A, lg, prepack=True, split_terms=3).double()
    b = _run_layer_rows(cfg, w, A, lg).double()
    assert bool(torch.isfinite(a).all()) and bool(torch.isfinite(b).all())
    row_l2 = ((a - b).norm(dim=1) / b.norm(dim=1).clamp_min(1e-30)).cpu().numpy()
    rms = float(b.pow(2).mean().sqrt())
    worst_el = float(((a - b).abs() / b.abs().clamp_min(max(rms, 1.0))).max())
    print(f"{name} T={T}: per-row relative L2 between the families: median {np.median(row_l2):.3e}, "
          f"worst {row_l2.max():.3e} (row {int(row_l2.argmax())}); worst element / rms {worst_el:.3e}")
    assert row_l2.max() <= 2e-3
    assert worst_el <= EXACT_SPLIT_MAX_ABS_TOL
    # the default arithmetic (three terms, then two) on every row as well
    c = _run_layer_rows(cfg, w, A, lg, prepack=True).double()
    row_l2 = ((c - b).norm(dim=1) / b.norm(dim=1).clamp_min(1e-30)).cpu().numpy()
    print(f"{name} T={T}: default terms against the raw-weight call: median {np.median(row_l2):.3e}, "
          f"worst {row_l2.max():.3e}")
    assert row_l2.max() <= 2e-3


# ---- the layer -------------------------------------------------------------------------

# The default arithmetic of the prepacked path (three FP6 terms in the first stage, two in
# the second) against the bf16-activation oracle: measured 5e-4 relative L2 and 3e-3 of the
# RMS for the worst element on the CPU model; a tenth of the contract is asserted.
DEFAULT_TERMS_MAX_ABS_TOL = 8e-3
DEFAULT_TERMS_REL_L2_TOL = 1e-3


def _check_prefill(cfg, T, w, A_bits, logits, terms=None, sample=128, wn=None, gpu_kw=None, cpu_kw=None,
                   block_size=None, contract_only=False):
    """terms: None = the library's default (3 terms in the first stage, 2 in the second),
    2 or 3 = that many in both."""
    gpu_kw = dict(gpu_kw or {})
    gpu_kw.update(prepack=True, split_terms=terms)
    g = cfgs._run_gpu(cfg, w, A_bits, logits, block_size, True, **gpu_kw)
    ids, tw = oracle.route_topk(logits, cfg.top_k, True)
    assert np.array_equal(g["ids"], ids) and np.array_equal(g["tw"].view(np.uint32), tw.view(np.uint32))
    rows = np.arange(T) if sample is None or sample >= T else \
        edge_tokens(g, T * cfg.top_k, cfg.top_k, sample, T)
    wn = w.numpy() if wn is None else wn
    c = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16, **(cpu_kw or {}))
    max_rel, rel_l2, nf = error_metrics(g["out"][rows], c["out"])
    # the default: 3 terms in the first stage, 2 in the second (3 where its sums are short)
    oracle.set_act_model(3 + 16 * (3 if cfg.I < 1024 else 2) if terms is None else terms)
    try:
        cm = cpu_layer(A_bits[rows], wn, ids[rows], tw[rows], threads=16, **(cpu_kw or {}))
    finally:
        oracle.set_act_model(0)
    m_rel, m_l2, m_nf = error_metrics(g["out"][rows], cm["out"])
    print(f"{cfg.name} T={T} terms={terms} rows checked {rows.size}: vs oracle max_abs/rms={max_rel:.3e} "
          f"rel_l2={rel_l2:.3e}; vs oracle with the same operands max_abs/rms={m_rel:.3e} rel_l2={m_l2:.3e}")
    assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL
    if not contract_only:
        assert m_nf and m_rel <= MODEL_MAX_ABS_TOL and m_l2 <= MODEL_REL_L2_TOL
    if terms == 3 and not contract_only:  # three terms: the bounds of the exact-split paths
        assert max_rel <= EXACT_SPLIT_MAX_ABS_TOL and rel_l2 <= EXACT_SPLIT_REL_L2_TOL
    if terms is None and not contract_only:
        assert max_rel <= DEFAULT_TERMS_MAX_ABS_TOL and rel_l2 <= DEFAULT_TERMS_REL_L2_TOL
    return g, wn


@pytest.mark.parametrize("terms", [None, 3, 2])
@pytest.mark.parametrize("T", [200, 513])
def test_config1_prepacked(T, terms):
    cfg = synth.CONFIGS["c1"]
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, 1900 + T)
    _check_prefill(cfg, T, w, A, lg, terms=terms)


def test_config2_zipf_prepacked():
    cfg = synth.CONFIGS["c2"]
    w = cfgs._weights(cfg)
    wn = None
    for T in (4096, 512):
        A, lg = cfgs._inputs(cfg, T, 2000)
        _, wn = _check_prefill(cfg, T, w, A, lg, wn=wn)


@pytest.mark.parametrize("T", [4096, 16384])
def test_config3_prepacked(T):
    cfg = synth.CONFIGS["c3"]
    w = cfgs._weights(cfg)
    A, lg = cfgs._inputs(cfg, T, 3000)
    g, wn = _check_prefill(cfg, T, w, A, lg, sample=160)
    assert np.all(np.isfinite(g["out"]))
    if T == 4096:   # the two- and the three-term options on the same inputs
        _check_prefill(cfg, T, w, A, lg, terms=2, sample=64, wn=wn)
        _check_prefill(cfg, T, w, A, lg, terms=3, sample=64, wn=wn)


@pytest.mark.parametrize("T", [1000, 8191])
def test_config4_prepacked(T):
    """Block scales of 2^+-20 and all-zero blocks: single terms dominate the outputs, so the
    end-to-end figure is held to the contract only (see the stage-wise tests of the raw path)."""
    cfg = synth.CONFIGS["c4"]
    key = ("c4x", 4000)
    if key not in cfgs._WEIGHTS:
        cfgs._WEIGHTS.clear()
        cfgs._WEIGHTS[key] = cfgs._extreme_weights(cfg, 4000)
    w = cfgs._WEIGHTS[key]
    A, lg = cfgs._inputs(cfg, T, 4000)
    _check_prefill(cfg, T, w, A, lg, contract_only=True)


@pytest.mark.parametrize("variant", ["bias", "limit", "bias_limit", "situ", "situ_bias"])
def test_epilogue_variants_prepacked(variant):
    """The first stage's epilogue is compiled per combination of bias, clamp and activation
    (a clamp that is off runs as a clamp at infinity next to a bias, SiTU without biases
    adds zeros): every combination that takes a different loop."""
    cfg = synth.CONFIGS["c1"]
    T, seed = 200, 1500
    w = cfgs._weights(cfg, seed)
    A, lg = cfgs._inputs(cfg, T, seed)
    b13 = (synth.rand_normal((cfg.E, 2 * cfg.I), seed, 21) * 0.5).astype(np.float32)
    b2 = (synth.rand_normal((cfg.E, cfg.H), seed, 22) * 0.5).astype(np.float32)
    gpu_kw, cpu_kw = {}, {}
    if "bias" in variant:
        gpu_kw.update(b13=to_dev(b13), b2=to_dev(b2))
        cpu_kw.update(b13=b13, b2=b2)
    if "limit" in variant:
        gpu_kw.update(swiglu_limit=1.5)
        cpu_kw.update(swiglu_limit=1.5)
    if "situ" in variant:
        gpu_kw.update(activation="situ", beta=3.0, linear_beta=20.0)
        cpu_kw.update(activation=1, beta=3.0, linear_beta=20.0)
    _check_prefill(cfg, T, w, A, lg, sample=48, gpu_kw=gpu_kw, cpu_kw=cpu_kw)


@pytest.mark.parametrize("bs", [16, 48, 64, 80, 128])
def test_block_sizes_prepacked(bs):
    cfg = synth.CONFIGS["c1"]
    T, seed = 160, 1700
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, seed)
    _check_prefill(cfg, T, w, A, lg, sample=48, block_size=bs)


def test_values_outside_the_range_prepacked():
    """inf/NaN codes and out-of-range scale bytes in some experts (flagged units: exact
    path) and rows with inf, NaN, huge and tiny values (flagged rows: their segments take
    the exact path); everything else on the fast path, in one call."""
    cfg = synth.MoEConfig("t", 256, 512, 8, 2, (300,), "uniform")
    T, seed = 300, 4300
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
    A[4, :] = 0
    g = cfgs._run_gpu(cfg, w, A, lg, None, True, prepack=True)
    ids, tw = oracle.route_topk(lg, cfg.top_k, True)
    c = cpu_layer(A, w.numpy(), ids, tw, threads=16)
    for t in range(T):   # row by row: the rows differ by many orders of magnitude
        max_rel, rel_l2, nf = error_metrics(g["out"][t], c["out"][t])
        assert nf and max_rel <= MAX_ABS_TOL and rel_l2 <= REL_L2_TOL, (t, max_rel, rel_l2)
    finite_rows = np.all(np.isfinite(c["out"]), axis=1)
    assert 0 < finite_rows.sum() < T


def test_expert_map_prepacked():
    cfg = synth.CONFIGS["c1"]
    T, seed = 300, 1800
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, seed)
    rng = np.random.default_rng(seed)
    local_n = cfg.E // 2
    owned = rng.permutation(cfg.E)[:local_n]
    emap = np.full(cfg.E, -1, dtype=np.int32)
    emap[owned] = np.arange(local_n, dtype=np.int32)
    own = to_dev(owned.astype(np.int64))
    fe = ve.FusedExperts(w.w13[own].contiguous(), w.w13_scale[own].contiguous(),
                         w.w2[own].contiguous(), w.w2_scale[own].contiguous(),
                         expert_map=to_dev(emap), local_num_experts=local_n,
                         scratch=ve.CaptureSafeScratch(), prepack=True)
    ids, tw = fe.route(to_dev(lg), cfg.top_k, True)
    out = fe.apply(to_dev(A, torch.bfloat16), ids, tw).cpu().numpy()
    ids_np, tw_np = ids.cpu().numpy(), tw.cpu().numpy()
    tw_local = np.where(emap[ids_np] >= 0, tw_np, np.float32(0.0)).astype(np.float32)
    c = cpu_layer(A, w.numpy(), ids_np, tw_local, threads=16)
    max_rel, rel_l2, nf = error_metrics(out, c["out"])
    assert nf and max_rel <= DEFAULT_TERMS_MAX_ABS_TOL and rel_l2 <= DEFAULT_TERMS_REL_L2_TOL, (max_rel, rel_l2)


def test_prepacked_calls_are_deterministic():
    """The packed path has no atomics: two calls give the same bits."""
    cfg = synth.CONFIGS["c1"]
    T = 300
    w = cfgs._weights(cfg, 1500)
    A, lg = cfgs._inputs(cfg, T, 1801)
    a = cfgs._run_gpu(cfg, w, A, lg, None, True, prepack=True)["out"]
    b = cfgs._run_gpu(cfg, w, A, lg, None, True, prepack=True)["out"]
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
