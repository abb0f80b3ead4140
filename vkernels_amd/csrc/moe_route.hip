// moe_route.hip — softmax -> top-k -> renormalise router, one wavefront per
// token.
//
// Semantics: src/python/vkernels/torch_ops/tokenspeed_amd/routing.py:59-157
// of the reference (no bias, scaling factor 1): p = softmax(logits) over the
// full row in fp32; top_k times the arg-max of p over the experts not yet
// taken, ties to the lowest expert index; weights p[ids], divided by their
// sum (a zero sum divides by 1).
//
// The selection compares rounded probabilities, so the arithmetic is fixed
// completely and the indices do not depend on the machine:
//   m      = max_e logits[e]
//   num[e] = route_exp(logits[e] - m)   fp32 mul, fma, round-to-even,
//                                       exponent add; 0 below -80
//   den    = lane l adds num[l], num[l+64], ... in ascending order, then six
//            butterfly steps v += v(lane ^ off), off = 32,16,8,4,2,1
//   p[e]   = num[e] / den               IEEE division
//   sum(w) = ((w0 + w1) + w2) + ...     selection order
// No multiply-add is contracted in this file; every fused operation is an
// explicit fmaf().
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vk_internal.hpp"

#pragma clang fp contract(off)

namespace vk {
namespace {

__device__ __forceinline__ float route_exp(float x) {
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

// PER = experts held per lane; covers E <= 64 * PER.
template <int PER>
__global__ __launch_bounds__(256) void route_topk_kernel(
    const float* __restrict__ logits, int T, int E, int top_k, int renormalize,
    int32_t* __restrict__ topk_ids, float* __restrict__ topk_w) {
  const int lane = threadIdx.x & 63;
  const int token = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (token >= T) return;  // whole wavefront leaves together
  const float* row = logits + (size_t)token * E;

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
  float my_w = 0.0f;
  int my_id = -1;
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
  if (lane < top_k) {
    topk_ids[(size_t)token * top_k + lane] = my_id;
    topk_w[(size_t)token * top_k + lane] = my_w;
  }
}

}  // namespace

void launch_route_topk(const float* logits, int T, int E, int top_k,
                       int renormalize, int32_t* topk_ids, float* topk_w,
                       hipStream_t stream) {
  const int waves_per_block = 4;
  const dim3 block(64 * waves_per_block);
  const dim3 grid((T + waves_per_block - 1) / waves_per_block);
#define VK_ROUTE_LAUNCH(PER)                                              \
  hipLaunchKernelGGL((route_topk_kernel<PER>), grid, block, 0, stream,    \
                     logits, T, E, top_k, renormalize, topk_ids, topk_w)
  if (E <= 64) VK_ROUTE_LAUNCH(1);
  else if (E <= 128) VK_ROUTE_LAUNCH(2);
  else if (E <= 256) VK_ROUTE_LAUNCH(4);
  else if (E <= 512) VK_ROUTE_LAUNCH(8);
  else VK_ROUTE_LAUNCH(16);
#undef VK_ROUTE_LAUNCH
}

}  // namespace vk
