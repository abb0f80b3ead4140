// moe_route.hpp — the router's per-token arithmetic, shared by the router kernel
// and the fused router + alignment kernel.  See moe_route.hip for the
// semantics and for why every operation is spelled out.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vk {

__device__ __forceinline__ float route_exp(float x) {
#pragma clang fp contract(off)
  if (!(x > -80.0f)) return 0.0f;
  const float t = x * 0x1.715476p+0f;       // fl32(log2 e)
  const float n = __builtin_rintf(t);       // round half to even
  float r = fmaf(n, -0x1.62e4p-1f, x);      // ln 2, high 16 bits
  r = fmaf(n, -0x1.7f7d1cp-20f, r);         // ln 2, remainder
  float p = 0x1.a01a02p-13f;                // 1/5040
  p = fmaf(p, r, 0x1.6c16c2p-10f);          // 1/720
  p = fmaf(p, r, 0x1.111112p-7f);           // 1/120
  p = fmaf(p, r, 0x1.555556p-5f);           // 1/24
  p = fmaf(p, r, 0x1.555556p-3f);           // 1/6
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  const int ni = (int)n;                    // in [-116, 0]
  return __uint_as_float(__float_as_uint(p) + ((uint32_t)ni << 23));
}

// One wavefront routes one token: `row` = its E logits.  PER = experts held per
// lane (E <= 64 * PER).  Lane sel < top_k returns the sel-th selection.
template <int PER>
__device__ __forceinline__ void route_token(const float* __restrict__ row, int E, int top_k,
                                            int renormalize, int lane, int& my_id, float& my_w) {
#pragma clang fp contract(off)
  float v[PER];
  float m = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? row[e] : -__builtin_inff();
    m = v[i] > m ? v[i] : m;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float o = __shfl_xor(m, off, 64);
    m = o > m ? o : m;
  }

  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? route_exp(v[i] - m) : 0.0f;
    s = s + v[i];
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s = s + __shfl_xor(s, off, 64);
  const float den = s;

  // key = probability bits : inverted expert index, 0 = not selectable.
  // Probabilities are non-negative, so their bit patterns order like the
  // values; the inverted index makes the lower expert win a tie.
  unsigned long long key[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    const float p = v[i] / den;
    key[i] = e < E ? (((unsigned long long)__float_as_uint(p) << 32) |
                      (unsigned long long)(0xFFFFFFFFu - (uint32_t)e))
                   : 0ull;
  }

  float wsum = 0.0f;
  my_w = 0.0f;
  my_id = -1;
  for (int sel = 0; sel < top_k; ++sel) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int i = 0; i < PER; ++i) best = key[i] > best ? key[i] : best;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const unsigned long long o = __shfl_xor(best, off, 64);
      best = o > best ? o : best;
    }
    const float w = __uint_as_float((uint32_t)(best >> 32));
    const int id = best ? (int)(0xFFFFFFFFu - (uint32_t)best) : -1;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (key[i] == best) key[i] = 0ull;  // keys are unique per expert
    wsum = sel == 0 ? w : wsum + w;
    if (lane == sel) {
      my_w = w;
      my_id = id;
    }
  }
  if (renormalize) {
    if (wsum == 0.0f) wsum = 1.0f;
    my_w = my_w / wsum;
  }
}

}  // namespace vk
