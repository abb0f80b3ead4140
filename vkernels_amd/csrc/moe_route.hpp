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

// The partner of every lane at the six levels of a wavefront-wide butterfly that runs
// off = 32, 16, 8, 4, 2, 1, without a trip through the LDS crossbar per level (a chain of
// ds_bpermute operations is what made a token cost four microseconds):
//   32, 16  v_permlane32_swap / v_permlane16_swap of a register with itself leave the two
//           halves (rows) side by side in two registers: lane l holds v[l & ~off] in the
//           first and v[l | off] in the second;
//   8       row_ror:8 is lane ^ 8 within a row of 16;
//   4       row_ror:4 is lane +- 4 within a row, which differs from lane ^ 4 only by a flip
//           of bit 3, and after the level before every value is the same in lanes l, l ^ 8;
//   2, 1    quad_perm [2,3,0,1] and [1,0,3,2].
// So each level combines exactly the two values that v(lane) and v(lane ^ off) would, the
// lower lane's first; with a commutative operation the result is, bit for bit, that of
// the butterfly written with six shuffles.  Every lane of the wavefront must be active.
template <class Op>
__device__ __forceinline__ uint32_t butterfly_u32(uint32_t v, Op op) {
  {
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    v = op(r[0], r[1]);
  }
  {
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = op(r[0], r[1]);
  }
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xF, 0xF, false));  // row_ror:8
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x124, 0xF, 0xF, false));  // row_ror:4
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
  return v;
}

// The same for a 64-bit value (both halves take the same way).
template <class Op>
__device__ __forceinline__ unsigned long long butterfly_u64(unsigned long long v, Op op) {
  auto join = [](uint32_t lo, uint32_t hi) { return ((unsigned long long)hi << 32) | lo; };
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  {
    const auto a = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
    const auto b = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
    v = op(join(a[0], b[0]), join(a[1], b[1]));
    lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  }
  {
    const auto a = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
    const auto b = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
    v = op(join(a[0], b[0]), join(a[1], b[1]));
    lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  }
#define VK_ROUTE_DPP_LEVEL(ctrl_)                                                                 \
  {                                                                                               \
    const uint32_t ol = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)lo, ctrl_, 0xF, 0xF, false); \
    const uint32_t oh = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)hi, ctrl_, 0xF, 0xF, false); \
    v = op(v, join(ol, oh));                                                                      \
    lo = (uint32_t)v, hi = (uint32_t)(v >> 32);                                                   \
  }
  VK_ROUTE_DPP_LEVEL(0x128)
  VK_ROUTE_DPP_LEVEL(0x124)
  VK_ROUTE_DPP_LEVEL(0x4E)
  VK_ROUTE_DPP_LEVEL(0xB1)
#undef VK_ROUTE_DPP_LEVEL
  return v;
}

// One wavefront routes NB tokens at once: rows[b] = the E logits of token b.  PER = experts
// held per lane (E <= 64 * PER).  Lane sel < top_k returns the sel-th selection of every
// token.  The tokens' arithmetic is independent, instruction by instruction, so the
// dependent chains of cross-lane steps of NB tokens can overlap where a wavefront has its
// SIMD to itself; where many wavefronts share a compute unit the instruction count is
// what costs, and NB = 1 is as fast.
template <int PER, int NB>
__device__ __forceinline__ void route_tokens(const float* const (&rows)[NB], int E, int top_k, int renormalize,
                                             int lane, int (&my_id)[NB], float (&my_w)[NB]) {
#pragma clang fp contract(off)
  float v[NB][PER];
  float m[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    m[b] = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + 64 * i;
      v[b][i] = e < E ? rows[b][e] : -__builtin_inff();
      m[b] = v[b][i] > m[b] ? v[b][i] : m[b];
    }
  }
#pragma unroll
  for (int b = 0; b < NB; ++b)
    m[b] = __uint_as_float(butterfly_u32(__float_as_uint(m[b]), [](uint32_t x, uint32_t y) {
      const float fx = __uint_as_float(x), fy = __uint_as_float(y);
      return __float_as_uint(fy > fx ? fy : fx);
    }));

  float den[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + 64 * i;
      v[b][i] = e < E ? route_exp(v[b][i] - m[b]) : 0.0f;
      s = s + v[b][i];
    }
    den[b] = s;
  }
  // (fp32 addition is commutative, so which of the two partners comes first does not matter)
#pragma unroll
  for (int b = 0; b < NB; ++b)
    den[b] = __uint_as_float(butterfly_u32(__float_as_uint(den[b]), [](uint32_t x, uint32_t y) {
      return __float_as_uint(__uint_as_float(x) + __uint_as_float(y));
    }));

  // key = probability bits : inverted expert index, 0 = not selectable.
  // Probabilities are non-negative, so their bit patterns order like the
  // values; the inverted index makes the lower expert win a tie.
  unsigned long long key[NB][PER];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + 64 * i;
      const float p = v[b][i] / den[b];
      key[b][i] = e < E ? (((unsigned long long)__float_as_uint(p) << 32) |
                           (unsigned long long)(0xFFFFFFFFu - (uint32_t)e))
                        : 0ull;
    }

  float wsum[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    wsum[b] = 0.0f;
    my_w[b] = 0.0f;
    my_id[b] = -1;
  }
  for (int sel = 0; sel < top_k; ++sel) {
    unsigned long long best[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      best[b] = 0ull;
#pragma unroll
      for (int i = 0; i < PER; ++i) best[b] = key[b][i] > best[b] ? key[b][i] : best[b];
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
      best[b] = butterfly_u64(best[b], [](unsigned long long x, unsigned long long y) { return y > x ? y : x; });
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const float w = __uint_as_float((uint32_t)(best[b] >> 32));
      const int id = best[b] ? (int)(0xFFFFFFFFu - (uint32_t)best[b]) : -1;
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if (key[b][i] == best[b]) key[b][i] = 0ull;  // keys are unique per expert
      wsum[b] = sel == 0 ? w : wsum[b] + w;
      if (lane == sel) {
        my_w[b] = w;
        my_id[b] = id;
      }
    }
  }
  if (renormalize) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (wsum[b] == 0.0f) wsum[b] = 1.0f;
      my_w[b] = my_w[b] / wsum[b];
    }
  }
}

// One wavefront routes one token: `row` = its E logits; lane sel < top_k returns the sel-th
// selection.
template <int PER>
__device__ __forceinline__ void route_token(const float* __restrict__ row, int E, int top_k,
                                            int renormalize, int lane, int& my_id, float& my_w) {
  const float* const rows[1] = {row};
  int ids[1];
  float ws[1];
  route_tokens<PER, 1>(rows, E, top_k, renormalize, lane, ids, ws);
  my_id = ids[0];
  my_w = ws[0];
}

}  // namespace vk
