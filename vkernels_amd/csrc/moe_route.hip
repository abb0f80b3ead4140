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

#include "moe_route.hpp"
#include "vk_internal.hpp"

#pragma clang fp contract(off)

namespace vk {
namespace {

// PER = experts held per lane; covers E <= 64 * PER.
template <int PER>
__global__ __launch_bounds__(256) void route_topk_kernel(
    const float* __restrict__ logits, int T, int E, int top_k, int renormalize,
    int32_t* __restrict__ topk_ids, float* __restrict__ topk_w) {
  const int lane = threadIdx.x & 63;
  const int token = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (token >= T) return;  // whole wavefront leaves together
  int my_id;
  float my_w;
  route_token<PER>(logits + (size_t)token * E, E, top_k, renormalize, lane, my_id, my_w);
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
