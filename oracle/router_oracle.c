/*
 * router_oracle.c — softmax / top-k / renormalise routing oracle.
 * TEST INFRASTRUCTURE ONLY (see moe_oracle.h).
 *
 * The reference has no CPU implementation of the router; its semantics come
 * from src/python/vkernels/torch_ops/tokenspeed_amd/routing.py:59-157 and
 * the formula in tests/python/test_tokenspeed_amd.py:517-537:
 *
 *   p      = softmax(logits)                      (fp32, full row)
 *   ids    = top_k times: argmax of p over the not-yet-selected experts,
 *            ties resolved to the LOWEST expert index (routing.py:112-118)
 *   w      = p[ids]
 *   w     /= sum(w)  (sum == 0 -> divide by 1)    (routing.py:120-123)
 *
 * Because the selection compares the rounded probabilities, two experts whose
 * logits differ by less than a rounding step of exp() can tie, and the tie
 * rule then decides the index.  For the indices to be reproducible bit for
 * bit on any machine the arithmetic is therefore pinned down completely:
 *
 *   m      = max_e logits[e]
 *   num[e] = vko_route_exp(logits[e] - m)          (below; only fp32 mul,
 *                                                    fma, rint, exponent add)
 *   den    = 64-lane tree sum: lane l first adds num[l], num[l+64], ... in
 *            ascending order (lanes past E hold 0), then six butterfly steps
 *            v[l] += v[l ^ off] for off = 32,16,8,4,2,1
 *   p[e]   = num[e] / den                          (IEEE fp32 division)
 *   sum(w) = ((w0 + w1) + w2) + ...                (selection order)
 *
 * Compile with -ffp-contract=off; every fused multiply-add is an explicit
 * fmaf().
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline float bits_to_float(uint32_t b) {
  float f;
  memcpy(&f, &b, sizeof f);
  return f;
}

static inline uint32_t float_to_bits(float f) {
  uint32_t b;
  memcpy(&b, &f, sizeof b);
  return b;
}

float vko_route_exp(float x) {
  /* exp underflows to exactly 0 below -80 so that the exponent add at the
   * end never leaves the normal range. */
  if (!(x > -80.0f)) return 0.0f;
  const float t = x * 0x1.715476p+0f;        /* fl32(log2 e)          */
  const float n = rintf(t);                  /* round half to even    */
  float r = fmaf(n, -0x1.62e4p-1f, x);       /* ln 2, high 16 bits    */
  r = fmaf(n, -0x1.7f7d1cp-20f, r);          /* ln 2, remainder       */
  float p = 0x1.a01a02p-13f;                 /* 1/5040                */
  p = fmaf(p, r, 0x1.6c16c2p-10f);           /* 1/720                 */
  p = fmaf(p, r, 0x1.111112p-7f);            /* 1/120                 */
  p = fmaf(p, r, 0x1.555556p-5f);            /* 1/24                  */
  p = fmaf(p, r, 0x1.555556p-3f);            /* 1/6                   */
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  const int32_t ni = (int32_t)n; /* in [-116, 0] */
  return bits_to_float(float_to_bits(p) + ((uint32_t)ni << 23));
}

void vko_route_topk(const float* logits, int T, int E, int top_k,
                    int renormalize, int32_t* topk_ids, float* topk_w) {
  float* p = (float*)malloc(sizeof(float) * (size_t)(E > 0 ? E : 1));
  for (int t = 0; t < T; ++t) {
    const float* row = logits + (size_t)t * E;
    float m = row[0];
    for (int e = 1; e < E; ++e)
      if (row[e] > m) m = row[e];
    for (int e = 0; e < E; ++e) p[e] = vko_route_exp(row[e] - m);

    float lane[64];
    for (int l = 0; l < 64; ++l) {
      float s = 0.0f;
      for (int e = l; e < E; e += 64) s = s + p[e];
      lane[l] = s;
    }
    for (int off = 32; off >= 1; off >>= 1) {
      float next[64];
      for (int l = 0; l < 64; ++l) next[l] = lane[l] + lane[l ^ off];
      memcpy(lane, next, sizeof lane);
    }
    const float den = lane[0];
    for (int e = 0; e < E; ++e) p[e] = p[e] / den;

    float wsum = 0.0f;
    for (int s = 0; s < top_k; ++s) {
      int best = -1;
      for (int e = 0; e < E; ++e) {
        if (p[e] < 0.0f) continue; /* already taken (marked below) */
        if (best < 0 || p[e] > p[best]) best = e;
      }
      topk_ids[(size_t)t * top_k + s] = best;
      const float w = best >= 0 ? p[best] : 0.0f;
      topk_w[(size_t)t * top_k + s] = w;
      wsum = (s == 0) ? w : wsum + w;
      if (best >= 0) p[best] = -1.0f;
    }
    if (renormalize) {
      if (wsum == 0.0f) wsum = 1.0f;
      for (int s = 0; s < top_k; ++s)
        topk_w[(size_t)t * top_k + s] = topk_w[(size_t)t * top_k + s] / wsum;
    }
  }
  free(p);
}
