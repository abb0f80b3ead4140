"""ctypes/numpy front end of liboracle.so (this repository's restatement) and,
when it has been built, of _ref/libvkref.so (the reference's own moe_fused.cpp
compiled as it lies).  TEST INFRASTRUCTURE ONLY.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

__all__ = [
    "HERE", "build", "lib", "ref_lib", "have_ref", "set_threads", "set_act_model", "act_model_block32",
    "fp4nib_to_f32bits", "ue8m0_to_float", "f32bits_to_bf16",
    "dequant_weight_tile", "moe_align_block_size",
    "moe_align_block_size_with_map", "align_max_em", "align_em_bound",
    "gather_sorted_weights", "fused_moe_mxfp4", "moe_gateup",
    "moe_act_epilogue", "moe_down", "moe_combine", "route_topk", "route_exp",
    "moe_layer",
    "aux_scale_byte", "mxfp4_moe_quant", "mxfp4_moe_sorted_quant", "mxfp4_moe_sort",
    "mxfp4_moe_sort_scales", "mxfp4_moe_scatter_reduce", "mxfp4_moe_scatter_reduce_q",
    "mxfp4_dequant_act",
]

HERE = Path(__file__).resolve().parent
_LIB = None
_REF = None

_c = ctypes
_P = ctypes.c_void_p


def build(ref: bool = True) -> None:
    """Compile liboracle.so (always) and _ref/libvkref.so (when the reference
    tree is present)."""
    subprocess.run(["make", "-s", "-C", str(HERE), "-B", "all"], check=True)
    if ref:
        subprocess.run(["make", "-s", "-C", str(HERE), "ref"], check=True)


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = HERE / "liboracle.so"
        if not path.is_file():
            subprocess.run(["make", "-s", "-C", str(HERE), "all"], check=True)
        _LIB = ctypes.CDLL(str(path))
        _LIB.vko_ue8m0_to_float.restype = _c.c_float
        _LIB.vko_fp4nib_to_f32bits.restype = _c.c_uint32
        _LIB.vko_f32bits_to_bf16.restype = _c.c_uint16
        _LIB.vko_f32bits_to_bf16.argtypes = [_c.c_uint32]
        _LIB.vko_align_max_em.restype = _c.c_size_t
        _LIB.vko_route_exp.restype = _c.c_float
        _LIB.vko_route_exp.argtypes = [_c.c_float]
        _LIB.vko_epilogue_value.restype = _c.c_float
        _LIB.vko_epilogue_value.argtypes = [_c.c_int] + [_c.c_float] * 5
    return _LIB


def ref_lib():
    """The compiled reference, or None when it has not been built."""
    global _REF
    if _REF is None:
        path = HERE / "_ref" / "libvkref.so"
        if not path.is_file():
            return None
        _REF = ctypes.CDLL(str(path))
    return _REF


def have_ref() -> bool:
    return ref_lib() is not None


def set_threads(n: int) -> None:
    lib().vko_set_threads(int(n))


def set_act_model(terms: int) -> None:
    """2 or 3: the GEMMs multiply the sum of that many FP6 (E2M3) terms per
    activation block of 32, the representation the GPU's prefill kernels use;
    0: the reference's arithmetic."""
    lib().vko_set_act_model(int(terms))


def act_model_block32(a_bits, terms: int = 2) -> np.ndarray:
    """The modelled values of one block of 32 bf16 bit patterns."""
    a = np.ascontiguousarray(a_bits, dtype=np.uint16)
    assert a.size == 32
    out = np.empty(32, dtype=np.float32)
    if int(terms) == 1:   # the W4A4 mode: quantised as mxfp4_moe_quant does, then dequantised
        lib().vko_aux_model_block32(_P(a.ctypes.data), _P(out.ctypes.data))
    else:
        lib().vko_act_model_block32(_P(a.ctypes.data), _P(out.ctypes.data), int(terms))
    return out


def _ptr(a):
    return None if a is None else _P(a.ctypes.data)


def _arr(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def _f(x):
    return _c.c_float(float(x))


# ---- scalar decoders ------------------------------------------------------

def fp4nib_to_f32bits(n: int) -> int:
    return int(lib().vko_fp4nib_to_f32bits(int(n)))


def ue8m0_to_float(s: int) -> float:
    return float(lib().vko_ue8m0_to_float(_c.c_uint8(int(s))))


def f32bits_to_bf16(b: int) -> int:
    return int(lib().vko_f32bits_to_bf16(int(b) & 0xFFFFFFFF))


def route_exp(x: float) -> float:
    return float(lib().vko_route_exp(float(x)))


def dequant_weight_tile(packed, scale, N, K, group_size=32, stride_packed=None,
                        stride_scale_n=None, stride_scale_k=1, which="lut", use_ref=False):
    """[K, N] uint16 bf16 tile.  which: 'lut' or 'ref' (the per-byte variant)."""
    packed = _arr(packed, np.uint8)
    scale = _arr(scale, np.uint8)
    stride_packed = K // 2 if stride_packed is None else stride_packed
    stride_scale_n = K // group_size if stride_scale_n is None else stride_scale_n
    out = np.zeros((K, N), dtype=np.uint16)
    if use_ref:
        fn = getattr(ref_lib(), "vkref_dequant_weight_tile" + ("_ref" if which == "ref" else ""))
    else:
        fn = getattr(lib(), "vko_dequant_weight_tile" + ("_ref" if which == "ref" else ""))
    fn(_ptr(packed), _ptr(scale), _ptr(out), N, K, group_size, stride_packed,
       stride_scale_n, stride_scale_k)
    return out


# ---- alignment --------------------------------------------------------------

def align_max_em(M, top_k, block_size, num_experts) -> int:
    return int(lib().vko_align_max_em(M, top_k, block_size, num_experts))


def align_em_bound(M, top_k, local_n, block_size) -> int:
    return int(lib().vko_align_em_bound(M, top_k, local_n, block_size))


def moe_align_block_size(topk_ids, block_size, num_experts, use_ref=False, fill=(None, None)):
    """Reference CPU semantics (EM may be 0; entries past EM keep `fill`)."""
    ids = _arr(topk_ids, np.int32)
    M, top_k = ids.shape
    max_em = align_max_em(M, top_k, block_size, num_experts)
    sids = np.full(max_em, M * top_k if fill[0] is None else fill[0], dtype=np.int32)
    eids = np.full(max(max_em // block_size, 1), -1 if fill[1] is None else fill[1], dtype=np.int32)
    fn = ref_lib().vkref_moe_align_block_size if use_ref else lib().vko_moe_align_block_size
    em = fn(_ptr(ids), M, top_k, block_size, num_experts, _ptr(sids), _ptr(eids))
    return sids, eids, int(em)


def moe_align_block_size_with_map(topk_ids_flat, num_experts, block_size, expert_map=None,
                                  local_n=None, max_EM=None):
    """Serving / device semantics: every one of the max_EM entries written,
    EM at least one block.  Returns (sorted_ids[max_EM], expert_ids[max_EM/bs], EM)."""
    ids = _arr(np.asarray(topk_ids_flat).ravel(), np.int32)
    n = ids.size
    local_n = num_experts if local_n is None else local_n
    if max_EM is None:
        max_EM = max(align_max_em(n, 1, block_size, local_n), block_size)
    emap = _arr(expert_map, np.int32)
    sids = np.full(max_EM, -12345, dtype=np.int32)
    eids = np.full(max_EM // block_size, -12345, dtype=np.int32)
    em = lib().vko_moe_align_block_size_with_map(_ptr(ids), _ptr(emap), n, block_size,
                                                 num_experts, local_n, max_EM,
                                                 _ptr(sids), _ptr(eids))
    return sids, eids, int(em)


def gather_sorted_weights(topk_w, sorted_ids):
    """topk_w_sorted[r] = topk_w.flat[sorted_ids[r]] (0 for padding rows), the
    gather the reference's tests do before calling the CPU oracle
    (tests/kernels/moe/test_moe_fused.cpp:703-709)."""
    w = np.asarray(topk_w, dtype=np.float32).ravel()
    sids = np.asarray(sorted_ids)
    out = np.zeros(sids.shape, dtype=np.float32)
    real = (sids >= 0) & (sids < w.size)
    out[real] = w[sids[real]]
    return out


# ---- the layer --------------------------------------------------------------

def fused_moe_mxfp4(A, w13, w13_scale, w2, w2_scale, sorted_ids, topk_w_sorted, expert_ids,
                    M, hidden, ispp, top_k, EM, *, out=None, act=None, group_size=32,
                    swiglu_limit=0.0, activation=0, beta=4.0, linear_beta=25.0,
                    b13=None, b2=None, use_ref=False):
    """Returns (out [M, hidden] fp32, act [EM, ispp] uint16)."""
    A = _arr(A, np.uint16); w13 = _arr(w13, np.uint8); w13_scale = _arr(w13_scale, np.uint8)
    w2 = _arr(w2, np.uint8); w2_scale = _arr(w2_scale, np.uint8)
    sids = _arr(sorted_ids, np.int32); eids = _arr(expert_ids, np.int32)
    tws = _arr(topk_w_sorted, np.float32)
    b13 = _arr(b13, np.float32); b2 = _arr(b2, np.float32)
    if out is None:
        out = np.zeros((M, hidden), dtype=np.float32)
    if act is None:
        act = np.zeros((max(EM, 1), ispp), dtype=np.uint16)
    fn = ref_lib().vkref_fused_moe_mxfp4 if use_ref else lib().vko_fused_moe_mxfp4
    fn(_ptr(A), _ptr(w13), _ptr(w13_scale), _ptr(w2), _ptr(w2_scale), _ptr(sids), _ptr(tws),
       _ptr(eids), _ptr(act), _ptr(out), M, hidden, ispp, top_k, EM, group_size,
       _f(swiglu_limit), activation, _f(beta), _f(linear_beta), _ptr(b13), _ptr(b2))
    return out, act


def moe_gateup(A, w13, w13_scale, sorted_ids, expert_ids, M, a_stride, k_base, hidden_k, ispp,
               top_k, EM, group_size=32, use_ref=False, fill=0.0):
    A = _arr(A, np.uint16); w13 = _arr(w13, np.uint8); w13_scale = _arr(w13_scale, np.uint8)
    sids = _arr(sorted_ids, np.int32); eids = _arr(expert_ids, np.int32)
    gu = np.full((EM, 2 * ispp), fill, dtype=np.float32)
    fn = ref_lib().vkref_moe_gateup if use_ref else lib().vko_moe_gateup
    fn(_ptr(A), _ptr(w13), _ptr(w13_scale), _ptr(sids), _ptr(eids), _ptr(gu), M, a_stride,
       k_base, hidden_k, ispp, top_k, EM, group_size)
    return gu


def moe_act_epilogue(gate_up, b13, sorted_ids, expert_ids, M, top_k, EM, ispp, swiglu_limit=0.0,
                     activation=0, beta=4.0, linear_beta=25.0, use_ref=False):
    gu = _arr(gate_up, np.float32); b13 = _arr(b13, np.float32)
    sids = _arr(sorted_ids, np.int32); eids = _arr(expert_ids, np.int32)
    act = np.zeros((EM, ispp), dtype=np.uint16)
    fn = ref_lib().vkref_moe_act_epilogue if use_ref else lib().vko_moe_act_epilogue
    fn(_ptr(gu), _ptr(b13), _ptr(act), _ptr(sids), _ptr(eids), M, top_k, EM, ispp,
       _f(swiglu_limit), activation, _f(beta), _f(linear_beta))
    return act


def moe_down(act, w2, w2_scale, sorted_ids, expert_ids, M, a_stride, k_base, ispp_k, hidden,
             top_k, EM, group_size=32, use_ref=False, fill=0.0):
    act = _arr(act, np.uint16); w2 = _arr(w2, np.uint8); w2_scale = _arr(w2_scale, np.uint8)
    sids = _arr(sorted_ids, np.int32); eids = _arr(expert_ids, np.int32)
    partial = np.full((EM, hidden), fill, dtype=np.float32)
    fn = ref_lib().vkref_moe_down if use_ref else lib().vko_moe_down
    fn(_ptr(act), _ptr(w2), _ptr(w2_scale), _ptr(sids), _ptr(eids), _ptr(partial), M, a_stride,
       k_base, ispp_k, hidden, top_k, EM, group_size)
    return partial


def moe_combine(partial, b2, topk_w_sorted, sorted_ids, expert_ids, M, hidden, top_k, EM,
                out=None, use_ref=False):
    partial = _arr(partial, np.float32); b2 = _arr(b2, np.float32)
    tws = _arr(topk_w_sorted, np.float32)
    sids = _arr(sorted_ids, np.int32); eids = _arr(expert_ids, np.int32)
    if out is None:
        out = np.zeros((M, hidden), dtype=np.float32)
    fn = ref_lib().vkref_moe_combine if use_ref else lib().vko_moe_combine
    fn(_ptr(partial), _ptr(b2), _ptr(tws), _ptr(sids), _ptr(eids), _ptr(out), M, hidden, top_k, EM)
    return out


# ---- MXFP4 MoE orchestration ops (moe_aux.cpp of the reference) -------------------

def _aux(name, use_ref):
    return getattr(ref_lib(), "vkref_" + name) if use_ref else getattr(lib(), "vko_" + name)


def aux_scale_byte(amax_bits: int) -> int:
    fn = lib().vko_aux_scale_byte
    fn.restype = _c.c_uint8
    return int(fn(_c.c_uint16(int(amax_bits) & 0x7FFF)))


def mxfp4_moe_quant(A, group_size=32, use_ref=False):
    """(packed [M, hidden/2], scales [M, hidden/group_size]) of bf16 rows A [M, hidden]."""
    A = _arr(A, np.uint16)
    M, hidden = A.shape
    packed = np.zeros((M, hidden // 2), dtype=np.uint8)
    scales = np.zeros((M, hidden // group_size), dtype=np.uint8)
    _aux("mxfp4_moe_quant", use_ref)(_ptr(A), _ptr(packed), _ptr(scales), M, hidden, group_size)
    return packed, scales


def mxfp4_moe_sorted_quant(A, sorted_ids, top_k, group_size=32, use_ref=False):
    A = _arr(A, np.uint16); sids = _arr(sorted_ids, np.int32)
    M, hidden = A.shape
    EM = sids.size
    packed = np.zeros((EM, hidden // 2), dtype=np.uint8)
    scales = np.zeros((EM, hidden // group_size), dtype=np.uint8)
    _aux("mxfp4_moe_sorted_quant", use_ref)(_ptr(A), _ptr(sids), _ptr(packed), _ptr(scales), M,
                                            hidden, group_size, top_k, EM)
    return packed, scales


def mxfp4_moe_sort(A, sorted_ids, top_k, use_ref=False):
    A = _arr(A, np.uint16); sids = _arr(sorted_ids, np.int32)
    M, hidden = A.shape
    out = np.zeros((sids.size, hidden), dtype=np.uint16)
    _aux("mxfp4_moe_sort", use_ref)(_ptr(A), _ptr(sids), _ptr(out), M, hidden, top_k, sids.size)
    return out


def mxfp4_moe_sort_scales(scales, sorted_ids, top_k, use_ref=False):
    scales = _arr(scales, np.uint8); sids = _arr(sorted_ids, np.int32)
    M, ng = scales.shape
    out = np.zeros((sids.size, ng), dtype=np.uint8)
    _aux("mxfp4_moe_sort_scales", use_ref)(_ptr(scales), _ptr(sids), _ptr(out), M, ng, top_k, sids.size)
    return out


def mxfp4_moe_scatter_reduce(partial, topk_w_sorted, sorted_ids, M, top_k, out=None, use_ref=False):
    partial = _arr(partial, np.float32); tws = _arr(topk_w_sorted, np.float32)
    sids = _arr(sorted_ids, np.int32)
    EM, width = partial.shape
    if out is None:
        out = np.zeros((M, width), dtype=np.float32)
    _aux("mxfp4_moe_scatter_reduce", use_ref)(_ptr(partial), _ptr(tws), _ptr(sids), _ptr(out), M,
                                              width, top_k, EM)
    return out


def mxfp4_moe_scatter_reduce_q(partial_q, partial_s, topk_w_sorted, sorted_ids, M, top_k,
                               group_size=32, out=None, use_ref=False):
    pq = _arr(partial_q, np.uint8); ps = _arr(partial_s, np.uint8)
    tws = _arr(topk_w_sorted, np.float32); sids = _arr(sorted_ids, np.int32)
    EM, width = pq.shape[0], pq.shape[1] * 2
    if out is None:
        out = np.zeros((M, width), dtype=np.float32)
    _aux("mxfp4_moe_scatter_reduce_q", use_ref)(_ptr(pq), _ptr(ps), _ptr(tws), _ptr(sids), _ptr(out),
                                                M, width, top_k, EM, group_size)
    return out


def mxfp4_dequant_act(packed, scales, group_size=32):
    """float32 values of quantised activations: table value x 2^(s-127), 0xFF -> 0
    (the W4A4 activation decode of tests/kernels/moe/test_moe_aux.cpp:53-69)."""
    packed = np.asarray(packed, dtype=np.uint8); scales = np.asarray(scales, dtype=np.uint8)
    table = np.array([fp4nib_to_f32bits(i) for i in range(16)], dtype=np.uint32).view(np.float32)
    nib = np.stack([packed & 15, packed >> 4], axis=-1).reshape(packed.shape[0], -1)
    sc = np.where(scales == 0xFF, np.float32(0.0),
                  (scales.astype(np.uint32) << 23).view(np.float32)).astype(np.float32)
    with np.errstate(invalid="ignore"):
        return table[nib] * np.repeat(sc, group_size, axis=1)


def route_topk(logits, top_k, renormalize=True):
    lg = _arr(logits, np.float32)
    T, E = lg.shape
    ids = np.zeros((T, top_k), dtype=np.int32)
    w = np.zeros((T, top_k), dtype=np.float32)
    lib().vko_route_topk(_ptr(lg), T, E, top_k, int(bool(renormalize)), _ptr(ids), _ptr(w))
    return ids, w


def moe_layer(A, logits, w13, w13_scale, w2, w2_scale, top_k, *, block_size=16, use_ref=False,
              threads=None, **kw):
    """Router -> align -> fused layer on the CPU.  Returns a dict with every
    intermediate the GPU path is compared against."""
    if threads is not None:
        set_threads(threads)
    A = _arr(A, np.uint16)
    M, hidden = A.shape
    E = w13.shape[0]
    ispp = w13.shape[1] // 2
    ids, w = route_topk(logits, top_k, True)
    sids, eids, em = moe_align_block_size(ids, 16, E, use_ref=use_ref)
    tws = gather_sorted_weights(w, sids[:max(em, 1)])
    out, act = fused_moe_mxfp4(A, w13, w13_scale, w2, w2_scale, sids, tws, eids, M, hidden, ispp,
                               top_k, em, use_ref=use_ref, **kw)
    return dict(topk_ids=ids, topk_w=w, sorted_ids=sids[:em], expert_ids=eids[:em // 16],
                EM=em, out=out, act=act[:em])
