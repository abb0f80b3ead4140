// moe_common.hpp — device helpers shared by the MoE GEMM translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxfp4.hpp"

namespace vk {

// Scale bytes the scaled-MFMA paths take (weights and activation blocks); units
// and rows outside go to the exact path.
constexpr uint32_t kScaleLo = 64u, kScaleHi = 190u;

// tanh for the SiTU epilogue: 1 - 2 / (1 + e^2x) with the
// hardware's exponential and reciprocal (+-1 at the infinities, NaN for NaN), and the
// series x - x^3/3 + 2 x^5/15 below |x| = 0.1, where the first form cancels (its error
// there is below 1e-8 relative).  A few ulp, far inside the bf16 rounding that follows.
__device__ __forceinline__ float tanh_fast(float x) {
  const float big = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * x));
  const float x2 = x * x;
  const float small = x * (1.0f - x2 * (0.33333334f - x2 * 0.13333334f));
  return fabsf(x) < 0.1f ? small : big;
}

// The SiTU activation (activation 1 of act_value; the reference's
// beta * tanh(g / beta) * sigmoid(g) * linear_beta * tanh(u / linear_beta), the second
// tanh left out when linear_beta <= 0) with those: inv_beta = 1 / beta,
// inv_linear_beta = 1 / linear_beta (unused when linear_beta <= 0).
__device__ __forceinline__ float situ_value(float g, float u, float beta, float inv_beta,
                                            float linear_beta, float inv_linear_beta) {
  // (below g = -87 the sigmoid is subnormal, which v_rcp_f32 flushes to zero: the
  // reciprocal is taken of the denominator scaled by 2^-64 and scaled back by a multiply)
  const float s = g < -87.0f ? 0x1p-64f : 1.0f;
  const float sig = __builtin_amdgcn_rcpf((1.0f + __expf(-g)) * s) * s;
  const float gate_out = beta * tanh_fast(g * inv_beta) * sig;
  const float up_out = linear_beta > 0.0f ? linear_beta * tanh_fast(u * inv_linear_beta) : u;
  return gate_out * up_out;
}

__device__ __forceinline__ float act_value(int activation, float g, float u,
                                           float limit, float beta,
                                           float linear_beta) {
  if (activation == 1)
    return situ_value(g, u, beta, __builtin_amdgcn_rcpf(beta), linear_beta,
                      linear_beta > 0.0f ? __builtin_amdgcn_rcpf(linear_beta) : 0.0f);
  if (limit > 0.0f) {
    if (g > limit) g = limit;
    if (u > limit) u = limit;
    if (u < -limit) u = -limit;
  }
  // v_exp_f32 / v_rcp_f32: about 1 ulp each, far inside the bf16 rounding that follows.
  // Below g = -87 the quotient is subnormal, which v_rcp_f32 flushes to zero (and an
  // infinite u then gives NaN where g / (1 + e^-g) * u is an infinity): there the
  // reciprocal is taken of the denominator scaled by 2^-64 and scaled back by a multiply.
  const float s = g < -87.0f ? 0x1p-64f : 1.0f;
  return (g * (__builtin_amdgcn_rcpf((1.0f + __expf(-g)) * s) * s)) * u;
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}


// Largest bf16 exponent field among the 8 values of v: the exponent of the
// largest magnitude, found with packed 16-bit maxima.
__device__ __forceinline__ uint32_t bf16x8_max_exponent(u32x4 v) {
  typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
  union { uint32_t u; u16x2 h; } a, b, c, d;
  a.u = v[0] & 0x7FFF7FFFu;
  b.u = v[1] & 0x7FFF7FFFu;
  c.u = v[2] & 0x7FFF7FFFu;
  d.u = v[3] & 0x7FFF7FFFu;
  a.h = __builtin_elementwise_max(a.h, b.h);
  c.h = __builtin_elementwise_max(c.h, d.h);
  a.h = __builtin_elementwise_max(a.h, c.h);
  const uint32_t m = max(a.u & 0xFFFFu, a.u >> 16);
  return m >> 7;
}

// s_waitcnt immediate that waits until at most n vector-memory operations are
// outstanding and for nothing else (vmcnt is split over bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

template <int N>
struct IntC {
  static constexpr int value = N;
};

// The DMA form of the global load: every lane's 16 (4) bytes at `src` go to LDS
// at byte address lds_base + 16 (4) * lane.  Written as assembly because the
// compiler makes every later LDS read wait for all DMA loads it has emitted
// itself, and for every register load issued along with them: a ring that is
// filled several steps ahead needs the counted waits of the kernel instead.
__device__ __forceinline__ void dma_load_16(const void* src, uint32_t lds_base) {
  __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :
                   : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(src)
                   : "memory");
}
__device__ __forceinline__ void dma_load_4(const void* src, uint32_t lds_base) {
  __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                   :
                   : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(src)
                   : "memory");
}

}  // namespace vk
