"""Host side of the fused MXFP4 MoE path: ctypes loader, capture-safe scratch,
EM bounds, and the `apply` call sequence of the serving integration.

Mirrors the interface of the reference's ``src/python/vkernels/vllm_experts.py``
for this path (same function names, arguments and error behaviour):

* :class:`CaptureSafeScratch`            vllm_experts.py:142-246
* :func:`max_num_tokens_hint`            vllm_experts.py:254-271
* :func:`max_em_count`                   vllm_experts.py:274-281
* :func:`moe_align_block_size_with_map`  vllm_experts.py:297-372
* :func:`find_libvkernels_hip`, :func:`load_libvkernels_hip`,
  :func:`resolve_moe_fn`, :func:`resolve_align_fn`   vllm_experts.py:381-459
* :func:`_align_em_bound`                vllm_experts.py:481-500
* :class:`FusedExperts.apply`            the kernel-facing part of
  ``VkernelFusedExperts.apply``, vllm_experts.py:813-1092 (the vLLM
  ``FusedMoE`` plumbing around it is not part of this path).

Every device operation goes through ``libvkernels_hip.so``; there is no CPU or
PyTorch fallback, and a missing library or symbol raises ``RuntimeError``.
PyTorch is used for tensor ownership and streams only.
"""
from __future__ import annotations

import ctypes
import importlib
import os

import numpy as np

from .native_runtime import find_library

__all__ = [
    "CaptureSafeScratch",
    "FusedExperts",
    "find_libvkernels_hip",
    "load_libvkernels_hip",
    "max_em_count",
    "max_num_tokens_hint",
    "moe_align_block_size_with_map",
    "resolve_align_fn",
    "resolve_moe_fn",
    "resolve_route_fn",
    "resolve_route_align_fn",
    "resolve_dequant_fn",
    "resolve_prepack_fns",
]

VK_OK = 0
VK_ERROR_INVALID_ARGUMENT = 1
VK_ERROR_OUT_OF_RANGE = 2
VK_ERROR_UNSUPPORTED = 3
VK_ERROR_INTERNAL = 4


def _require_torch():
    try:
        return importlib.import_module("torch")
    except ImportError as exc:  # pragma: no cover
        raise ImportError("vkernels_amd.vllm_experts needs torch for tensor operations") from exc


def _default_capture_probe() -> bool:
    """True while a graph capture is active on the current stream."""
    try:
        torch = importlib.import_module("torch")
        return bool(torch.cuda.is_available() and torch.cuda.is_current_stream_capturing())
    except Exception:  # noqa: BLE001 - "not capturing" when it cannot be asked
        return False


class CaptureSafeScratch:
    """Persistent device buffers that are sized once and sliced afterwards.

    The device entry points allocate nothing; their scratch (``act_scratch``,
    ``out``, ``sorted_ids``, ``expert_ids``) belongs to the caller and must
    keep its address across graph replays.  ``get`` allocates a ``(device,
    key)`` buffer at ``capacity`` the first time, returns ``store[:count]``
    afterwards, grows it when a larger count arrives outside a capture and
    raises ``RuntimeError`` when that happens during one (the captured graph
    still points at the old storage).
    """

    def __init__(self, capture_probe=None):
        self._buffers = {}
        self._capture_probe = capture_probe or _default_capture_probe

    def keys(self):
        return list(self._buffers.keys())

    def get(self, key, count: int, *, dtype, device, capacity: int | None = None,
            name: str = "scratch"):
        if count < 0:
            raise ValueError(f"{name}: count must be non-negative, got {count}")
        slot = (device.index, key)
        store = self._buffers.get(slot)
        if store is not None and store.numel() >= count:
            return store[:count]
        if self._capture_probe():
            have = 0 if store is None else store.numel()
            raise RuntimeError(
                f"[vkernels] persistent {name} (dev={device.index}, key={key!r}, cap={have}) "
                f"is too small for {count} elements AND a graph capture is active - refusing "
                f"to grow (the captured graph references the old storage). Size it on the "
                f"eager warm-up run with a larger max-token budget.")
        torch = _require_torch()
        cap = count if capacity is None else max(count, capacity)
        store = torch.empty(cap, dtype=dtype, device=device)
        self._buffers[slot] = store
        return store[:count]

    def reset(self) -> None:
        self._buffers.clear()


def max_num_tokens_hint() -> int:
    """Token budget used to size persistent scratch: MAX_NUM_BATCHED_TOKENS,
    VLLM_MAX_NUM_BATCHED_TOKENS, else 8192."""
    for var in ("MAX_NUM_BATCHED_TOKENS", "VLLM_MAX_NUM_BATCHED_TOKENS"):
        raw = os.environ.get(var)
        if not raw:
            continue
        try:
            n = int(raw)
        except ValueError:
            continue
        if n > 0:
            return n
    return 8192


def max_em_count(max_M: int, top_k: int, local_n: int) -> int:
    """High-water mark of EM: M*top_k + local experts, rounded up to 64."""
    return (max_M * top_k + local_n + 63) // 64 * 64


def _local_n(local_num_experts, global_num_experts) -> int:
    return local_num_experts if local_num_experts and local_num_experts > 0 else global_num_experts


def _align_em_bound(M: int, top_k: int, local_n: int, block_size: int) -> int:
    """Host upper bound on EM for any routing of M*top_k indices over local_n
    experts: one block per expert that can be hit, plus the rest in one
    expert.  A constant per batch shape, so grids sized by it are capture-safe."""
    n = M * top_k
    if n <= 0:
        return block_size
    head = min(n, local_n) * block_size
    if n <= local_n:
        return head
    return head + (n - local_n + block_size - 1) // block_size * block_size


def moe_align_block_size_with_map(topk_ids_flat, num_experts: int, block_size: int,
                                  expert_map=None):
    """Host alignment with optional global->local expert remap.

    Returns ``(sorted_ids[EM], expert_ids[EM // block_size], EM)``: flat
    indices grouped by ascending local expert (ascending within an expert),
    every expert padded to a multiple of ``block_size`` with the sentinel
    ``N = len(topk_ids_flat)``; ``expert_ids`` is the local expert of each
    block; ``EM`` is at least ``block_size`` (all-padding block, expert -1)
    when nothing routes.  Entries mapped to -1 are dropped.
    """
    ids = np.ascontiguousarray(topk_ids_flat, dtype=np.int32).ravel()
    n = ids.size
    # Same skip rules as the device kernel: ids outside [0, num_experts) and
    # ids mapped to a negative local expert are dropped.
    valid = (ids >= 0) & (ids < num_experts)
    local = np.full(n, -1, dtype=np.int64)
    if expert_map is not None:
        emap = np.asarray(expert_map, dtype=np.int64)
        local[valid] = emap[ids[valid].astype(np.int64)]
    else:
        local[valid] = ids[valid]
    flat = np.nonzero(local >= 0)[0]
    order = flat[np.argsort(local[flat], kind="stable")]
    experts, counts = np.unique(local[flat], return_counts=True)
    padded = (counts + block_size - 1) // block_size * block_size
    em = int(padded.sum())
    if em == 0:
        return (np.full(block_size, n, dtype=np.int32), np.full(1, -1, dtype=np.int32), block_size)
    starts = np.concatenate(([0], np.cumsum(padded)[:-1]))
    sorted_ids = np.full(em, n, dtype=np.int32)
    first = np.concatenate(([0], np.cumsum(counts)[:-1]))
    # position of the i-th routed entry (in expert order) inside the padded layout
    dest = np.repeat(starts - first, counts) + np.arange(order.size)
    sorted_ids[dest] = order
    expert_ids = np.repeat(experts, padded // block_size).astype(np.int32)
    return sorted_ids, expert_ids, em


# ---------------------------------------------------------------------------
# library loading
# ---------------------------------------------------------------------------

_lib_cache: dict = {}


def find_libvkernels_hip():
    return find_library(("libvkernels_hip.so",))


def load_libvkernels_hip():
    """Load and cache ``libvkernels_hip.so``; RuntimeError when absent."""
    if "lib" not in _lib_cache:
        path = find_libvkernels_hip()
        if path is None:
            raise RuntimeError(
                "libvkernels_hip.so not found. Set VKERNELS_LIB to its path or build it in "
                "tree with `python -m vkernels_amd.build`.")
        _lib_cache["lib"] = ctypes.CDLL(path)
    return _lib_cache["lib"]


_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float

_MOE_ARGTYPES = [_P] * 9 + [_I] * 4 + [_P, _P, _I, _F, _I, _F, _F, _P, _P, _I, _P]
_ALIGN_ARGTYPES = [_P, _P] + [_I] * 6 + [_P] * 4
_ROUTE_ARGTYPES = [_P, _I, _I, _I, _I, _P, _P, _P]
_DEQUANT_ARGTYPES = [_P, _P, _P] + [_I] * 7 + [_P]


def resolve_moe_fn(lib):
    """``vk_hip_fused_moe_mxfp4`` or RuntimeError (the CPU ABI's
    ``vk_fused_moe_mxfp4`` has another signature and is never a stand-in)."""
    fn = getattr(lib, "vk_hip_fused_moe_mxfp4", None)
    if fn is None:
        raise RuntimeError("vk_hip_fused_moe_mxfp4 not found in libvkernels_hip.so")
    fn.restype = None
    fn.argtypes = _MOE_ARGTYPES
    return fn


def resolve_moe_ws_fn(lib):
    """(``vk_hip_fused_moe_mxfp4_ws``, ``vk_hip_fused_moe_mxfp4_workspace_bytes``), the fused
    call with a caller-owned workspace, or (None, None) when the library predates it."""
    fn = getattr(lib, "vk_hip_fused_moe_mxfp4_ws", None)
    size_fn = getattr(lib, "vk_hip_fused_moe_mxfp4_workspace_bytes", None)
    if fn is None or size_fn is None:
        return None, None
    fn.restype = None
    fn.argtypes = _MOE_ARGTYPES[:-1] + [_P, ctypes.c_size_t, _P]
    size_fn.restype = ctypes.c_size_t
    size_fn.argtypes = [_I, _I, _I, _I, _I]
    return fn, size_fn


MOE_OVERWRITE_OUT = 1  # VK_HIP_MOE_OVERWRITE_OUT
MOE_SPLIT2 = 2         # VK_HIP_MOE_SPLIT2
MOE_W4A4 = 4           # VK_HIP_MOE_W4A4
MOE_SPLIT3 = 8         # VK_HIP_MOE_SPLIT3


def resolve_prepack_fns(lib):
    """(vk_hip_moe_prepack_bytes, vk_hip_moe_prepack_weights, vk_hip_fused_moe_mxfp4_prepacked)
    or (None, None, None) when the library predates them."""
    size_fn = getattr(lib, "vk_hip_moe_prepack_bytes", None)
    pack_fn = getattr(lib, "vk_hip_moe_prepack_weights", None)
    moe_fn = getattr(lib, "vk_hip_fused_moe_mxfp4_prepacked", None)
    if size_fn is None or pack_fn is None or moe_fn is None:
        return None, None, None
    size_fn.restype = ctypes.c_size_t
    size_fn.argtypes = [_I, _I, _I, _I]
    pack_fn.restype = _I
    pack_fn.argtypes = [_P, _P, _I, _I, _I, _I, _P, ctypes.c_size_t, _P]
    moe_fn.restype = None
    moe_fn.argtypes = _MOE_ARGTYPES[:-1] + [_P, ctypes.c_size_t, ctypes.c_uint, _P, _P, _I, _P]
    return size_fn, pack_fn, moe_fn


def resolve_moe_ex_fn(lib):
    """``vk_hip_fused_moe_mxfp4_ex`` (workspace and flags) or None."""
    fn = getattr(lib, "vk_hip_fused_moe_mxfp4_ex", None)
    if fn is None:
        return None
    fn.restype = None
    fn.argtypes = _MOE_ARGTYPES[:-1] + [_P, ctypes.c_size_t, ctypes.c_uint, _P]
    return fn


def resolve_align_fn(lib):
    """``vk_hip_moe_align_block_size`` or None when the symbol is absent."""
    fn = getattr(lib, "vk_hip_moe_align_block_size", None)
    if fn is None:
        return None
    fn.restype = _I
    fn.argtypes = _ALIGN_ARGTYPES
    return fn


def resolve_route_fn(lib):
    fn = getattr(lib, "vk_hip_moe_route_topk", None)
    if fn is None:
        raise RuntimeError("vk_hip_moe_route_topk not found in libvkernels_hip.so")
    fn.restype = _I
    fn.argtypes = _ROUTE_ARGTYPES
    return fn


def resolve_route_align_fn(lib):
    """vk_hip_moe_route_align (router and alignment, one launch for decode-sized batches)."""
    fn = getattr(lib, "vk_hip_moe_route_align", None)
    if fn is None:
        raise RuntimeError("vk_hip_moe_route_align not found in libvkernels_hip.so")
    fn.restype = _I
    fn.argtypes = [_P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _P, _P, _P, _P, _P]
    return fn


def resolve_route_layer_fn(lib):
    """vk_hip_moe_route_layer_mxfp4: router, alignment and the layer behind one call."""
    try:
        fn = lib.vk_hip_moe_route_layer_mxfp4
    except AttributeError:
        return None
    fn.restype = _I
    fn.argtypes = ([_P] * 10 + [_I] * 6 + [_P, _I, _I, _I, _P, _P, _P, _F, _I, _F, _F, _P, _P, _P,
                                           ctypes.c_size_t, ctypes.c_uint, _P, _P, _I, _P])
    return fn


def resolve_dequant_fn(lib):
    fn = getattr(lib, "vk_hip_dequant_weight_tile", None)
    if fn is None:
        raise RuntimeError("vk_hip_dequant_weight_tile not found in libvkernels_hip.so")
    fn.restype = _I
    fn.argtypes = _DEQUANT_ARGTYPES
    return fn


def last_error(lib) -> str:
    lib.vk_last_error.restype = ctypes.c_char_p
    return (lib.vk_last_error() or b"").decode()


def _check(lib, status: int, what: str) -> None:
    if status != VK_OK:
        raise RuntimeError(f"{what} failed with status {status}: {last_error(lib)}")


def _ptr(t):
    return _P(0) if t is None else _P(t.data_ptr())


def _stream(torch):
    return _P(torch.cuda.current_stream().cuda_stream)


_scratch = CaptureSafeScratch()


def default_block_size(M: int, top_k: int | None = None, lib=None, packed_experts: int = 0,
                       hidden: int = 0, ispp: int = 0) -> int:
    """The reference's policy: 16-row alignment for decode batches, 64 above
    (vllm_experts.py:846).  With top_k given the library is asked what its kernels
    like best (vk_hip_moe_default_block_size: 16 while M * top_k routed rows run the
    decode kernels, blocks of 128 for the tile kernels' windows beyond; packed_experts,
    hidden, ispp: the number of local experts and the layer's widths of a caller that gives
    the prepacked weights, for whom the decode kernels' range follows the rows per expert)."""
    if top_k is not None:
        lib = load_libvkernels_hip() if lib is None else lib
        fn = getattr(lib, "vk_hip_moe_default_block_size", None)
        if fn is None:
            raise RuntimeError("the loaded libvkernels_hip has no vk_hip_moe_default_block_size; "
                               "pass block_size, or call default_block_size(M) for the reference's policy")
        if packed_experts > 0:
            fn = lib.vk_hip_moe_default_block_size_ex
            fn.restype, fn.argtypes = _I, [_I, _I, _I, _I, _I]
            return int(fn(int(M), int(top_k), int(packed_experts), int(hidden), int(ispp)))
        fn.restype, fn.argtypes = _I, [_I, _I]
        return int(fn(int(M), int(top_k)))
    return 16 if M <= 32 else 64


# ---- launch shapes: candidates, the tuning store, queries (vkernels_hip.h) ----
def moe_tile_candidates(stage: int, lib=None) -> list[tuple[int, int, int, int]]:
    """(variant, wavefronts, tiles, depth) of every shape the stage can be launched at."""
    lib = load_libvkernels_hip() if lib is None else lib
    fn = lib.vk_hip_moe_tile_candidates
    fn.restype, fn.argtypes = _I, [_I, _P, _I]
    n = int(fn(stage, None, 0))
    buf = (ctypes.c_int * (4 * n))()
    fn(stage, buf, n)
    return [tuple(buf[4 * i:4 * i + 4]) for i in range(n)]


def moe_tile_query(stage: int, K: int, ncols: int, n_flat: int, lib=None, packed: bool = False,
                   block_size: int = 16):
    """((variant, wavefronts, tiles, depth), from_store) a call of this size is planned with
    (packed: when the caller gives the prepacked weights; block_size 32: ... in blocks of 32)."""
    lib = load_libvkernels_hip() if lib is None else lib
    fn = lib.vk_hip_moe_tile_query
    fn.restype, fn.argtypes = _I, [_I, _I, _I, _I, _P]
    buf = (ctypes.c_int * 4)()
    stored = int(fn(stage + ((4 if block_size == 32 else 2) if packed else 0), K, ncols, n_flat, buf))
    return tuple(buf), bool(stored)


def moe_tile_set(stage: int, K: int, ncols: int, n_flat: int, shape, lib=None) -> None:
    """Puts (shape None: removes) the record of this problem in the process's tuning store."""
    lib = load_libvkernels_hip() if lib is None else lib
    fn = lib.vk_hip_moe_tile_set
    fn.restype, fn.argtypes = _I, [_I, _I, _I, _I, _P]
    buf = None if shape is None else (ctypes.c_int * 4)(*shape)
    if fn(stage, K, ncols, n_flat, buf) != VK_OK:
        raise ValueError(last_error(lib))


def moe_tuning_load(directory: str | None = None, lib=None) -> int:
    lib = load_libvkernels_hip() if lib is None else lib
    fn = lib.vk_hip_moe_tuning_load
    fn.restype, fn.argtypes = _I, [ctypes.c_char_p]
    return int(fn(None if directory is None else os.fsencode(directory)))


def moe_tuning_dump(lib=None) -> str:
    """The process's tuning store as the text of a moe_fused.gfx950.tune file."""
    lib = load_libvkernels_hip() if lib is None else lib
    fn = lib.vk_hip_moe_tuning_dump
    fn.restype, fn.argtypes = ctypes.c_size_t, [ctypes.c_char_p, ctypes.c_size_t]
    need = int(fn(None, 0))
    buf = ctypes.create_string_buffer(need)
    fn(buf, need)
    return buf.value.decode()


class FusedExperts:
    """The kernel-facing call sequence of the serving integration on torch
    device tensors: (route ->) align on device -> fused layer, all enqueued on
    the current stream with no host synchronisation.

    Weights keep the raw serving layout: ``w13`` [E, 2*I, H/2] uint8 with gate
    rows first, ``w2`` [E, H, I/2] uint8, ue8m0 scales [.., K/32] uint8.
    ``prepack=True`` adds the prepacked form (1.0625 x the bytes of codes and scales);
    with ``keep_raw=False`` the raw tensors are let go of after the packing and every
    call runs on the prepacked form alone.
    """

    def __init__(self, w13, w13_scale, w2, w2_scale, *, b13=None, b2=None, activation="swiglu",
                 swiglu_limit: float = 0.0, beta: float = 4.0, linear_beta: float = 25.0,
                 expert_map=None, local_num_experts=None, scratch: CaptureSafeScratch | None = None,
                 prepack: bool = False, split_terms: int | None = None, w4a4: bool = False,
                 keep_raw: bool = True):
        torch = _require_torch()
        self.torch = torch
        self.lib = load_libvkernels_hip()
        self.moe_fn = resolve_moe_fn(self.lib)
        self.moe_ws_fn, self.ws_bytes_fn = resolve_moe_ws_fn(self.lib)
        self.moe_ex_fn = resolve_moe_ex_fn(self.lib)
        self.align_fn = resolve_align_fn(self.lib)
        if self.align_fn is None:
            raise RuntimeError("vk_hip_moe_align_block_size not found in libvkernels_hip.so")
        self.route_fn = resolve_route_fn(self.lib)
        self.route_align_fn = resolve_route_align_fn(self.lib)
        self.route_layer_fn = resolve_route_layer_fn(self.lib)
        for name, t in (("w13", w13), ("w13_scale", w13_scale), ("w2", w2), ("w2_scale", w2_scale)):
            if t.dtype != torch.uint8 or not t.is_contiguous() or not t.is_cuda:
                raise ValueError(f"{name} must be a contiguous uint8 device tensor")
        E, n2, hk = w13.shape
        self.E, self.ispp, self.hidden = E, n2 // 2, hk * 2
        if tuple(w2.shape) != (E, self.hidden, self.ispp // 2):
            raise ValueError("w2 shape does not match w13")
        if tuple(w13_scale.shape) != (E, n2, self.hidden // 32) or \
                tuple(w2_scale.shape) != (E, self.hidden, self.ispp // 32):
            raise ValueError("scale shapes must be [.., K/32]")
        if self.hidden % 64 or self.ispp % 64:
            raise ValueError("hidden and ispp must be multiples of 64")
        self.w13, self.w13_scale, self.w2, self.w2_scale = w13, w13_scale, w2, w2_scale
        self.b13, self.b2 = b13, b2
        # hand the library a workspace (VKERNELS_MOE_WORKSPACE=0: the plain entry point)
        self.use_workspace = os.environ.get("VKERNELS_MOE_WORKSPACE", "1") != "0"
        self.activation = {"swiglu": 0, "situ": 1}[activation] if isinstance(activation, str) \
            else int(activation)
        self.swiglu_limit, self.beta, self.linear_beta = swiglu_limit, beta, linear_beta
        self.expert_map = expert_map
        self.local_n = _local_n(local_num_experts, E)
        # routing indices are global: with a map, as many experts as the map has entries
        self.global_E = E if expert_map is None else int(expert_map.numel())
        if expert_map is not None and (expert_map.dtype != torch.int32 or not expert_map.is_cuda):
            raise ValueError("expert_map must be an int32 device tensor")
        self.scratch = scratch or _scratch
        # a second copy of the weights in the layout of the prefill-sized kernels
        # (load time; batches of more than 512 routed rows then run at the FP4 rate)
        if split_terms not in (None, 2, 3):
            raise ValueError("split_terms must be None (three FP6 terms in the first stage, two in the "
                             "second), 2 or 3 (that many in both)")
        self.split_terms = split_terms
        # W4A4: batches of more than 512 routed rows quantise their activations to MXFP4 as
        # the reference's mxfp4_moe_quant does (needs the prepacked weights)
        self.w4a4 = bool(w4a4)
        if self.w4a4 and not prepack:
            raise ValueError("w4a4=True needs prepack=True")
        self.w13_packed = self.w2_packed = None
        self.moe_prepacked_fn = None
        if not keep_raw and not prepack:
            raise ValueError("keep_raw=False needs prepack=True")
        if prepack:
            self.prepack()
        if not keep_raw:
            # One copy of the weights: every kernel family reads the prepacked form (the
            # decode kernels their packed instantiations, the exact paths the raw codes a
            # flagged unit keeps), so the references to the raw tensors are dropped here
            # and the calls pass null for them.  The caller drops its own to free the memory.
            if not self.use_workspace or self.moe_prepacked_fn is None:
                raise RuntimeError("keep_raw=False needs the workspace entry points")
            torch.cuda.current_stream().synchronize()  # the packing kernels have read them
            self.w13 = self.w13_scale = self.w2 = self.w2_scale = None

    def block_size_for(self, M: int, top_k: int) -> int:
        """The alignment block the library's kernels like best for M tokens on these weights
        (with prepacked weights the library is told how many experts they hold)."""
        return default_block_size(M, top_k, self.lib,
                                  packed_experts=self.local_n if self.w13_packed is not None else 0,
                                  hidden=self.hidden, ispp=self.ispp)

    def prepack(self):
        """Build the prepacked copies of w13 and w2 (idempotent)."""
        if self.w13_packed is not None:
            return
        torch = self.torch
        size_fn, pack_fn, moe_fn = resolve_prepack_fns(self.lib)
        if pack_fn is None:
            raise RuntimeError("vk_hip_moe_prepack_weights not found in libvkernels_hip.so")
        packed = []
        for stage, (w, ws, rows, K) in enumerate(((self.w13, self.w13_scale, 2 * self.ispp, self.hidden),
                                                  (self.w2, self.w2_scale, self.hidden, self.ispp))):
            n = int(size_fn(self.E, rows, K, stage))
            buf = torch.empty(n, dtype=torch.uint8, device=w.device)
            st = pack_fn(_ptr(w), _ptr(ws), self.E, rows, K, stage, _ptr(buf), n, _stream(torch))
            _check(self.lib, st, "vk_hip_moe_prepack_weights")
            packed.append(buf)
        self.w13_packed, self.w2_packed = packed
        self.moe_prepacked_fn = moe_fn

    # -- routing ------------------------------------------------------------
    def route(self, logits, top_k: int, renormalize: bool = True):
        torch = self.torch
        T, E = logits.shape
        logits = logits.contiguous()
        ids = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
        w = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
        st = self.route_fn(_ptr(logits), T, E, top_k, int(renormalize), _ptr(ids), _ptr(w),
                           _stream(torch))
        _check(self.lib, st, "vk_hip_moe_route_topk")
        return ids, w

    # -- alignment ------------------------------------------------------------
    def align(self, topk_ids, block_size: int, num_experts: int | None = None,
              max_tokens: int | None = None):
        """Returns (sorted_ids[max_EM], expert_ids[max_EM/bs], out_EM[1], max_EM)."""
        torch = self.torch
        M, top_k = topk_ids.shape
        dev = topk_ids.device
        if block_size <= 0 or block_size % 16 != 0:
            raise ValueError(f"block_size must be a positive multiple of 16, got {block_size}")
        num_experts = self.global_E if num_experts is None else num_experts
        max_em = _align_em_bound(M, top_k, self.local_n, block_size)
        cap_m = max(M, max_tokens or 0)
        cap = _align_em_bound(cap_m, top_k, self.local_n, block_size)
        sids = self.scratch.get(("sids", block_size), max_em, dtype=torch.int32, device=dev,
                                capacity=cap, name="sorted_ids")
        eids = self.scratch.get(("eids", block_size), max_em // block_size, dtype=torch.int32,
                                device=dev, capacity=cap // block_size, name="expert_ids")
        out_em = self.scratch.get("out_em", 1, dtype=torch.int32, device=dev, name="out_em")
        st = self.align_fn(_ptr(topk_ids), _ptr(self.expert_map), M, top_k, block_size,
                           num_experts, self.local_n, max_em, _ptr(sids), _ptr(eids),
                           _ptr(out_em), _stream(torch))
        _check(self.lib, st, "vk_hip_moe_align_block_size")
        return sids, eids, out_em, max_em

    def route_align(self, logits, top_k: int, renormalize: bool = True, block_size: int | None = None,
                    max_tokens: int | None = None):
        """route() and align() through the library's one call (one launch for decode-sized
        batches).  Returns (topk_ids, topk_w, sorted_ids, expert_ids, out_EM, max_EM,
        block_size); logits' E columns are the experts the expert map speaks of."""
        torch = self.torch
        T, E = logits.shape
        dev = logits.device
        block_size = self.block_size_for(T, top_k) if block_size is None else block_size
        if block_size <= 0 or block_size % 16 != 0:
            raise ValueError(f"block_size must be a positive multiple of 16, got {block_size}")
        logits = logits.contiguous()
        ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
        w = torch.empty((T, top_k), dtype=torch.float32, device=dev)
        max_em = _align_em_bound(T, top_k, self.local_n, block_size)
        cap = _align_em_bound(max(T, max_tokens or 0), top_k, self.local_n, block_size)
        sids = self.scratch.get(("sids", block_size), max_em, dtype=torch.int32, device=dev,
                                capacity=cap, name="sorted_ids")
        eids = self.scratch.get(("eids", block_size), max_em // block_size, dtype=torch.int32,
                                device=dev, capacity=cap // block_size, name="expert_ids")
        out_em = self.scratch.get("out_em", 1, dtype=torch.int32, device=dev, name="out_em")
        st = self.route_align_fn(_ptr(logits), T, E, top_k, int(renormalize), _ptr(self.expert_map),
                                 block_size, self.local_n, max_em, _ptr(ids), _ptr(w), _ptr(sids),
                                 _ptr(eids), _ptr(out_em), _stream(torch))
        _check(self.lib, st, "vk_hip_moe_route_align")
        return ids, w, sids, eids, out_em, max_em, block_size

    # -- the layer --------------------------------------------------------------
    def apply(self, hidden_states, topk_ids, topk_weights=None, *, block_size: int | None = None,
              max_tokens: int | None = None, out_fp32=None, output_dtype=None, aligned=None):
        """hidden_states [M, H] bf16, topk_ids [M, k] int32, topk_weights [M, k]
        fp32 (None = ones).  Returns the fp32 [M, H] result, or, with output_dtype
        (say torch.bfloat16, what the reference's apply hands back,
        src/python/vkernels/vllm_experts.py:1092), that result cast.
        aligned = (sorted_ids, expert_ids, max_EM) of route_align() / align() for this
        block_size: the alignment is then not made again."""
        torch = self.torch
        M, K = hidden_states.shape
        if K != self.hidden:
            raise ValueError(f"hidden size {K} does not match the weights ({self.hidden})")
        top_k = topk_ids.shape[1]
        dev = hidden_states.device
        block_size = self.block_size_for(M, top_k) if block_size is None else block_size
        if block_size <= 0 or block_size % 16 != 0:
            raise ValueError(f"block_size must be a positive multiple of 16, got {block_size}")
        hidden_states = hidden_states.contiguous()
        topk_ids = topk_ids.to(torch.int32).contiguous()
        if topk_weights is None:
            topk_weights = self.scratch.get("ones", M * top_k, dtype=torch.float32, device=dev,
                                            capacity=(max_tokens or M) * top_k).view(M, top_k)
            topk_weights.fill_(1.0)
        topk_weights = topk_weights.to(torch.float32).contiguous()
        if out_fp32 is None:
            out_fp32 = torch.empty((M, K), dtype=torch.float32, device=dev)
        # with the flags entry point the library clears `out` inside its first stage
        overwrite = self.moe_ex_fn is not None and self.use_workspace and M > 0
        if not overwrite:
            out_fp32.zero_()
        if M > 0:
            if aligned is None:
                sids, eids, _, max_em = self.align(topk_ids, block_size, max_tokens=max_tokens)
            else:
                sids, eids, max_em = aligned
            self.fused_call(hidden_states, topk_ids, topk_weights, sids, eids, max_em, block_size,
                            out_fp32, max_tokens=max_tokens, overwrite=overwrite)
        return out_fp32 if output_dtype is None else out_fp32.to(output_dtype)

    def fused_call(self, hidden_states, topk_ids, topk_weights, sids, eids, max_em: int,
                   block_size: int, out_fp32, *, max_tokens: int | None = None,
                   overwrite: bool = False):
        """The C call of apply() alone: accumulates the layer into out_fp32 (overwrite=True:
        writes it, whatever it held) for rows already aligned (sids, eids, max_em from
        align()).  Scratch comes from self.scratch."""
        torch = self.torch
        M, K = hidden_states.shape
        top_k = topk_ids.shape[1]
        dev = hidden_states.device
        cap = _align_em_bound(max(M, max_tokens or 0), top_k, self.local_n, block_size)
        act = self.scratch.get(("act", self.ispp), max_em * self.ispp, dtype=torch.bfloat16,
                               device=dev, capacity=cap * self.ispp, name="act_scratch")
        args = (_ptr(hidden_states), _ptr(self.w13), _ptr(self.w13_scale), _ptr(self.w2),
                _ptr(self.w2_scale), _ptr(topk_ids), _ptr(topk_weights), _ptr(act),
                _ptr(out_fp32), M, K, self.ispp, top_k, _ptr(sids), _ptr(eids), max_em,
                float(self.swiglu_limit), self.activation, float(self.beta),
                float(self.linear_beta), _ptr(self.b13), _ptr(self.b2), block_size)
        # the entry points return void: a refused call (contract violation, launch error)
        # leaves its message in the thread's error state, which is read back here
        self.lib.vk_set_last_error(0, b"")
        if self.moe_ws_fn is not None and self.use_workspace:
            # the library splits the rows once per call into this workspace where its
            # tile kernels run (large batches, large K); held like the other scratch
            # (sized once at the token budget)
            need = int(self.ws_bytes_fn(M, K, self.ispp, top_k, max_em))
            cap_bytes = int(self.ws_bytes_fn(max(M, max_tokens or 0), K, self.ispp, top_k, cap))
            ws = self.scratch.get(("ws", K, self.ispp), need, dtype=torch.uint8, device=dev,
                                  capacity=cap_bytes, name="workspace")
            flags = MOE_OVERWRITE_OUT if overwrite else 0
            if self.w13_packed is not None:
                if self.w4a4:
                    flags |= MOE_W4A4
                elif self.split_terms == 2:
                    flags |= MOE_SPLIT2
                elif self.split_terms == 3:
                    flags |= MOE_SPLIT3
                self.moe_prepacked_fn(*args, _ptr(ws), need, flags, _ptr(self.w13_packed),
                                      _ptr(self.w2_packed), self.E, _stream(torch))
            elif self.moe_ex_fn is not None:
                self.moe_ex_fn(*args, _ptr(ws), need, flags, _stream(torch))
            elif overwrite:
                raise RuntimeError("overwrite=True needs vk_hip_fused_moe_mxfp4_ex")
            else:
                self.moe_ws_fn(*args, _ptr(ws), need, _stream(torch))
        elif overwrite:
            raise RuntimeError("overwrite=True needs the workspace entry points")
        else:
            self.moe_fn(*args, _stream(torch))
        if int(self.lib.vk_last_error_code()) != VK_OK:
            raise RuntimeError(f"fused MoE call refused: {last_error(self.lib)}")

    def route_layer(self, hidden_states, router_logits, top_k: int, *, renormalize: bool = True,
                    block_size: int | None = None, max_tokens: int | None = None, out_fp32=None):
        """Router, alignment and the layer through the library's one call
        (vk_hip_moe_route_layer_mxfp4: two launches for a handful of tokens, the router's,
        the alignment's and the layer's otherwise).  Returns (out fp32 [M, H], topk_ids,
        topk_w, sorted_ids, expert_ids, out_EM, max_EM); `out` is written whatever it held."""
        torch = self.torch
        if self.route_layer_fn is None:
            raise RuntimeError("vk_hip_moe_route_layer_mxfp4 not found in libvkernels_hip.so")
        M, K = hidden_states.shape
        if K != self.hidden:
            raise ValueError(f"hidden size {K} does not match the weights ({self.hidden})")
        E = router_logits.shape[1]
        dev = hidden_states.device
        block_size = self.block_size_for(M, top_k) if block_size is None else block_size
        if block_size <= 0 or block_size % 16 != 0:
            raise ValueError(f"block_size must be a positive multiple of 16, got {block_size}")
        hidden_states = hidden_states.contiguous()
        logits = router_logits.contiguous()
        ids = torch.empty((M, top_k), dtype=torch.int32, device=dev)
        w = torch.empty((M, top_k), dtype=torch.float32, device=dev)
        max_em = _align_em_bound(M, top_k, self.local_n, block_size)
        cap = _align_em_bound(max(M, max_tokens or 0), top_k, self.local_n, block_size)
        sids = self.scratch.get(("sids", block_size), max_em, dtype=torch.int32, device=dev,
                                capacity=cap, name="sorted_ids")
        eids = self.scratch.get(("eids", block_size), max_em // block_size, dtype=torch.int32,
                                device=dev, capacity=cap // block_size, name="expert_ids")
        out_em = self.scratch.get("out_em", 1, dtype=torch.int32, device=dev, name="out_em")
        act = self.scratch.get(("act", self.ispp), max_em * self.ispp, dtype=torch.bfloat16,
                               device=dev, capacity=cap * self.ispp, name="act_scratch")
        need = int(self.ws_bytes_fn(M, K, self.ispp, top_k, max_em))
        cap_bytes = int(self.ws_bytes_fn(max(M, max_tokens or 0), K, self.ispp, top_k, cap))
        ws = self.scratch.get(("ws", K, self.ispp), need, dtype=torch.uint8, device=dev,
                              capacity=cap_bytes, name="workspace")
        if out_fp32 is None:
            out_fp32 = torch.empty((M, K), dtype=torch.float32, device=dev)
        flags = MOE_OVERWRITE_OUT
        if self.w13_packed is not None:
            flags |= MOE_W4A4 if self.w4a4 else MOE_SPLIT2 if self.split_terms == 2 else \
                MOE_SPLIT3 if self.split_terms == 3 else 0
        st = self.route_layer_fn(
            _ptr(hidden_states), _ptr(logits), _ptr(self.w13), _ptr(self.w13_scale), _ptr(self.w2),
            _ptr(self.w2_scale), _ptr(ids), _ptr(w), _ptr(act), _ptr(out_fp32), M, E, K, self.ispp, top_k,
            int(renormalize), _ptr(self.expert_map), self.local_n, block_size, max_em, _ptr(sids), _ptr(eids),
            _ptr(out_em), float(self.swiglu_limit), self.activation, float(self.beta), float(self.linear_beta),
            _ptr(self.b13), _ptr(self.b2), _ptr(ws), need, flags, _ptr(self.w13_packed), _ptr(self.w2_packed),
            self.E, _stream(torch))
        _check(self.lib, st, "vk_hip_moe_route_layer_mxfp4")
        return out_fp32, ids, w, sids, eids, out_em, max_em

    def forward(self, hidden_states, router_logits, top_k: int, **kw):
        """Router + layer: returns (out fp32 [M, H], topk_ids, topk_w)."""
        if self.route_layer_fn is not None and self.use_workspace and not kw:
            out, ids, w = self.route_layer(hidden_states, router_logits, top_k)[:3]
            return out, ids, w
        ids, w = self.route(router_logits, top_k, True)
        return self.apply(hidden_states, ids, w, **kw), ids, w
