"""Seeded synthetic inputs for the fused MXFP4 MoE layer.

Everything integer-valued (weight codes, scale bytes, routing tables) comes
from a counter-based splitmix64 generator written with torch integer ops, so
the same seed gives the same bytes on the CPU and on the GPU and for any
library version.  Floating-point inputs (activations, logits) are drawn on the
CPU in float64 and rounded once.

Weight conventions (src/c/vkernels/kernels/moe_fused.hpp:56-66 of the
reference): w13 [E, 2*I, H/2] uint8 with gate rows [0, I) and up rows [I, 2I),
w2 [E, H, I/2] uint8, low nibble = even k; scales [.., K/32] uint8 ue8m0.
Codes are drawn from the 12 finite E2M1 codes {0..5, 8..13}: codes 6, 7, 14,
15 decode to inf/NaN in the reference's table
(src/c/vkernels/kernels/moe_fused.cpp:24-39) and are used only by the
robustness cases, as in tests/python/test_mxfp4_serving_parity.py:102-105.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch

FINITE_CODES = (0, 1, 2, 3, 4, 5, 8, 9, 10, 11, 12, 13)

_MASK64 = (1 << 64) - 1


def _s64(v: int) -> int:
    """Two's-complement view of a 64-bit constant as a Python int for int64."""
    v &= _MASK64
    return v - (1 << 64) if v >= (1 << 63) else v


_GOLDEN = _s64(0x9E3779B97F4A7C15)
_MUL1 = _s64(0xBF58476D1CE4E5B9)
_MUL2 = _s64(0x94D049BB133111EB)


def _lsr(x: torch.Tensor, n: int) -> torch.Tensor:
    return (x >> n) & ((1 << (64 - n)) - 1)


def splitmix64(counter: torch.Tensor) -> torch.Tensor:
    """splitmix64 output function applied to an int64 counter tensor."""
    z = counter + _GOLDEN
    z = (z ^ _lsr(z, 30)) * _MUL1
    z = (z ^ _lsr(z, 27)) * _MUL2
    return z ^ _lsr(z, 31)


def _stream_base(seed: int, stream: int) -> int:
    """Start counter of an independent stream: a hash of (seed, stream)."""
    z = (seed * 0xD1342543DE82EF95 + stream * 0xAF251AF3B0F025B5 + 0x1234567) & _MASK64
    z ^= z >> 29
    z = (z * 0xBF58476D1CE4E5B9) & _MASK64
    z ^= z >> 32
    return _s64(z)


def rand_u63(n: int, seed: int, stream: int, device="cpu", offset: int = 0) -> torch.Tensor:
    """n non-negative pseudo-random int64 values (63 bits)."""
    idx = torch.arange(offset, offset + n, dtype=torch.int64, device=device)
    return splitmix64(idx + _stream_base(seed, stream)) & ((1 << 63) - 1)


def rand_codes_packed(shape, seed: int, stream: int, device="cpu",
                      codes=FINITE_CODES, chunk: int = 1 << 24) -> torch.Tensor:
    """uint8 tensor of `shape`; each byte packs two codes drawn from `codes`."""
    n = int(math.prod(shape))
    table = torch.tensor(codes, dtype=torch.int64, device=device)
    out = torch.empty(n, dtype=torch.uint8, device=device)
    for off in range(0, n, chunk):
        m = min(chunk, n - off)
        r = rand_u63(m, seed, stream, device, off)
        lo = table[(r >> 8) % len(codes)]
        hi = table[(r >> 32) % len(codes)]
        out[off:off + m] = (lo | (hi << 4)).to(torch.uint8)
    return out.reshape(shape)


def rand_bytes(shape, lo: int, hi: int, seed: int, stream: int, device="cpu",
               chunk: int = 1 << 24) -> torch.Tensor:
    """uint8 tensor uniform in [lo, hi]."""
    n = int(math.prod(shape))
    out = torch.empty(n, dtype=torch.uint8, device=device)
    for off in range(0, n, chunk):
        m = min(chunk, n - off)
        r = rand_u63(m, seed, stream, device, off)
        out[off:off + m] = (lo + (r >> 16) % (hi - lo + 1)).to(torch.uint8)
    return out.reshape(shape)


def rand_normal(shape, seed: int, stream: int, std: float = 1.0) -> np.ndarray:
    """float64 N(0, std^2) samples (Box-Muller on the CPU)."""
    n = int(math.prod(shape))
    r1 = rand_u63(n, seed, stream, "cpu").numpy().astype(np.float64)
    r2 = rand_u63(n, seed, stream + 1000003, "cpu").numpy().astype(np.float64)
    u1 = (r1 + 1.0) / float(1 << 63)
    u2 = r2 / float(1 << 63)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * std).reshape(shape)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit patterns (uint16)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    b = b + 0x7FFF + ((b >> 16) & 1)
    return (b >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


@dataclass
class MoEWeights:
    w13: torch.Tensor        # [E, 2I, H/2] uint8
    w13_scale: torch.Tensor  # [E, 2I, H/32] uint8
    w2: torch.Tensor         # [E, H, I/2] uint8
    w2_scale: torch.Tensor   # [E, H, I/32] uint8

    @property
    def nbytes(self) -> int:
        return sum(t.numel() for t in (self.w13, self.w13_scale, self.w2, self.w2_scale))

    def expert_bytes(self) -> int:
        return self.nbytes // self.w13.shape[0]

    def to(self, device) -> "MoEWeights":
        return MoEWeights(*(t.to(device) for t in
                            (self.w13, self.w13_scale, self.w2, self.w2_scale)))

    def numpy(self):
        return tuple(t.cpu().numpy() for t in
                     (self.w13, self.w13_scale, self.w2, self.w2_scale))


def make_weights(E: int, H: int, I: int, seed: int, device="cpu",
                 scale_lo: int = 123, scale_hi: int = 129,
                 codes=FINITE_CODES) -> MoEWeights:
    """MXFP4 expert weights: uniform codes, scale exponents uniform in
    [scale_lo-127, scale_hi-127] (default [-4, 2])."""
    return MoEWeights(
        rand_codes_packed((E, 2 * I, H // 2), seed, 1, device, codes),
        rand_bytes((E, 2 * I, H // 32), scale_lo, scale_hi, seed, 2, device),
        rand_codes_packed((E, H, I // 2), seed, 3, device, codes),
        rand_bytes((E, H, I // 32), scale_lo, scale_hi, seed, 4, device),
    )


def make_activations(T: int, H: int, seed: int) -> np.ndarray:
    """[T, H] bf16 bit patterns of N(0,1) samples."""
    return f32_to_bf16_bits(rand_normal((T, H), seed, 5).astype(np.float32))


def make_logits(kind: str, T: int, E: int, seed: int, A_bits: np.ndarray | None = None,
                H: int | None = None) -> np.ndarray:
    """[T, E] fp32 router logits.

    uniform : N(0,1) per entry
    zipf    : N(0,1) + log of a Zipf(s=1.1) popularity over a seeded expert
              permutation (load imbalance)
    router  : A @ Wr^T with Wr ~ N(0, 0.02) [E, H], fp32
    """
    if kind == "uniform":
        return rand_normal((T, E), seed, 6).astype(np.float32)
    if kind == "zipf":
        base = rand_normal((T, E), seed, 6)
        rank = np.argsort(rand_u63(E, seed, 7).numpy(), kind="stable")
        pop = np.empty(E, dtype=np.float64)
        pop[rank] = 1.0 / np.power(np.arange(1, E + 1, dtype=np.float64), 1.1)
        return (base + np.log(pop / pop.sum())[None, :]).astype(np.float32)
    if kind == "router":
        assert A_bits is not None and H is not None
        wr = rand_normal((E, H), seed, 8, std=0.02).astype(np.float32)
        return (bf16_bits_to_f32(A_bits).astype(np.float32) @ wr.T).astype(np.float32)
    raise ValueError(kind)


@dataclass(frozen=True)
class MoEConfig:
    name: str
    H: int
    I: int
    E: int
    top_k: int
    Ts: tuple
    logits: str


# The five benchmark configurations.
CONFIGS = {
    "c0": MoEConfig("c0", 256, 512, 8, 2, (16,), "router"),
    "c1": MoEConfig("c1", 2880, 2880, 32, 4, (1, 8, 32, 64), "uniform"),
    "c2": MoEConfig("c2", 2880, 2880, 128, 4, (64, 512, 4096), "zipf"),
    "c3": MoEConfig("c3", 7168, 2048, 256, 8, (4096, 16384), "uniform"),
    "c4": MoEConfig("c4", 4096, 1536, 64, 6, (1, 7, 33, 255, 1000, 8191), "uniform"),
}


def config_seed(cfg: MoEConfig, T: int) -> int:
    return int(cfg.name[1:]) * 1000 + T


def algorithmic_bytes(H: int, I: int, E: int, top_k: int, T: int, active_experts: int) -> int:
    """HBM bytes one layer call has to move: each active expert's packed
    weights and scales once, activations in, logits in, act out and back in,
    fp32 output."""
    per_expert = (2 * I * H // 2) + (2 * I * H // 32) + (H * I // 2) + (H * I // 32)
    return (active_experts * per_expert + 2 * T * H + 4 * T * E
            + 2 * 2 * T * top_k * I + 4 * T * H)


def algorithmic_flops(H: int, I: int, top_k: int, T: int) -> int:
    return 6 * T * top_k * H * I
