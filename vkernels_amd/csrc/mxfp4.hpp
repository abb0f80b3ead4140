// mxfp4.hpp — device-side decode of packed E2M1 weights with ue8m0 scales.
//
// The decode table is the reference's, not OCP-MXFP4: code -> {0, .25, 1,
// 1.5, 2, 3, inf, NaN} with the sign in bit 3
// (src/c/vkernels/kernels/moe_fused.cpp:24-39); scale byte s -> 2^(s-127),
// 0xFF -> 0, 0 -> 2^-127 (moe_fused.cpp:50-64); the product is rounded to
// bf16 (moe_fused.cpp:41-45, a no-op for every finite product because the
// codes carry one mantissa bit).
//
// Two routines produce the same bf16 bits:
//   dequant8_exact  integer construction, valid for every code and scale
//                   byte, including the reference's NaN sign quirks;
//   dequant8_fast   gfx950's v_cvt_scalef32_pk_bf16_fp4, valid when no code
//                   is inf/NaN and the scale byte lies in [3, 252].
// The hardware conversion decodes OCP E2M1 {0, .5, 1, 1.5, 2, 3, 4, 6}.  The
// reference's finite values are exactly half of the OCP values of the codes
// {0, 1, 4, 5, 6, 7}, so the fast path adds 2 to every code whose exponent
// field is non-zero and halves the scale (s-1 instead of s).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
// The same four floats at an address that is only 4-byte aligned (a caller's bias row, a
// view into a larger buffer): global memory takes multi-dword accesses at dword alignment.
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// One code -> the fp32 bits of the reference's decode table
// (src/c/vkernels/kernels/moe_fused.cpp:24-39): +-{0, .25, 1, 1.5, 2, 3, inf}, NaN.
__device__ __forceinline__ uint32_t fp4nib_to_f32bits(uint32_t nib) {
  const uint32_t sign = (nib & 8u) << 28;
  const uint32_t e = (nib >> 1) & 3u, m = nib & 1u;
  if (e == 0u) return m ? (sign | 0x3E800000u) : sign;
  if (e == 3u) return m ? 0x7FC00000u : (sign | 0x7F800000u);
  return sign | ((126u + e) << 23) | (m << 22);
}

// One code with one scale byte -> bf16 bits, every case of the reference's
// fp32 multiply-then-round reproduced with integers.
__device__ __forceinline__ uint32_t dequant1_exact(uint32_t nib, uint32_t s) {
  const uint32_t c3 = nib & 7u;
  const uint32_t sgn = (nib & 8u) << 12;
  if (c3 == 0u) return sgn;                    // +-0 * anything finite
  if (c3 == 7u) return 0x7FC0u;                // NaN keeps the table's payload
  if (c3 == 6u) return s == 0xFFu ? 0xFFC0u    // inf * 0: x86 default NaN
                                  : (sgn | 0x7F80u);
  if (s == 0xFFu) return sgn;                  // finite * 0
  const int ec = (c3 == 1u) ? -2 : (int)(c3 >> 1) - 1;
  const uint32_t m = (c3 == 1u) ? 0u : (c3 & 1u);
  const int ex = ec + (int)s;                  // bf16 exponent field
  if (ex >= 255) return sgn | 0x7F80u;         // fp32 overflow -> inf
  if (ex >= 1) return sgn | ((uint32_t)ex << 7) | (m << 6);
  return sgn | ((m ? 96u : 64u) >> (-ex));     // bf16 subnormal, still exact
}

// Eight codes (one dword, low nibble first) with one scale byte -> 8 bf16.
__device__ __forceinline__ u32x4 dequant8_exact(uint32_t x, uint32_t s) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t lo = dequant1_exact((x >> (8 * i)) & 15u, s);
    const uint32_t hi = dequant1_exact((x >> (8 * i + 4)) & 15u, s);
    r[i] = lo | (hi << 16);
  }
  return r;
}

// Codes whose exponent field is non-zero move up by 2 (01m -> 10m, 10m -> 11m).
__device__ __forceinline__ uint32_t fp4x8_to_ocp_doubled(uint32_t x) {
  return x + ((x | (x >> 1)) & 0x22222222u);
}

// Non-zero where a code of x is inf or NaN (both exponent bits set).
__device__ __forceinline__ uint32_t fp4x8_nonfinite(uint32_t x) {
  return x & (x >> 1) & 0x22222222u;
}

// True when the fast path decodes scale byte s exactly: the halved scale
// 2^(s-128) is a normal float and no product leaves bf16's normal range.
__device__ __forceinline__ bool scale_fast_ok(uint32_t s) {
  return (s - 3u) <= 249u;
}

// fp32 whose value is 2^(s-128), the halved scale of the fast path.
__device__ __forceinline__ float scale_half_f32(uint32_t s) {
  return __uint_as_float((s - 1u) << 23);
}

__device__ __forceinline__ u32x4 dequant8_fast(uint32_t x, float scale_half) {
  const uint32_t y = fp4x8_to_ocp_doubled(x);
  union { bf16x2 v; uint32_t u; } c0, c1, c2, c3;
  c0.v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(y, scale_half, 0);
  c1.v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(y, scale_half, 1);
  c2.v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(y, scale_half, 2);
  c3.v = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(y, scale_half, 3);
  u32x4 r = {c0.u, c1.u, c2.u, c3.u};
  return r;
}

// fp32 -> bf16 bits, round to nearest even with no NaN special case
// (moe_fused.cpp:41-45).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t b = __float_as_uint(f);
  b += 0x7FFFu + ((b >> 16) & 1u);
  return b >> 16;
}

}  // namespace vk
