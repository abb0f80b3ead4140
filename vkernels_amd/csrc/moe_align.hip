// moe_align.hip — on-device moe_align_block_size: stable bucket of the flat
// routing indices by (local) expert, each expert padded to a multiple of
// block_size.
//
// Output contract (src/c/vkernels/kernels/moe_fused.hpp:346-390 and
// moe_fused.hip:1983-2071 of the reference): sorted_ids holds, per local
// expert in ascending order, the flat indices token*top_k+sel routed to it in
// ascending order, padded with N = M*top_k; expert_ids holds the local expert
// of every block, -1 for blocks past the end; every entry up to max_EM is
// written; *out_EM is the padded row count, at least one block.
//
// One launch, one workgroup per local expert, no scratch memory and no limit
// on N.  Workgroup e
//   1. histograms all N indices into LDS (every workgroup needs the counts
//      of the experts before it) while each of its wavefronts counts the
//      entries of expert e in its own contiguous slice of the indices;
//   2. sums the padded counts of the experts before it (its first row) and
//      of all experts (EM);
//   3. walks its slices again and writes the matching flat indices in
//      order, ranked with ballot + popcount;
//   4. pads its last block, writes its expert_ids and its share of the
//      sentinel tail [EM, max_EM).
// The routing table is read from L2 by every workgroup, and every workgroup
// builds the whole histogram; for the largest benchmark shape (N = 131072,
// 256 experts) that is 256 x 512 KiB of L2 reads and 75 us, against a layer
// that takes milliseconds.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "moe_route.hpp"
#include "vk_internal.hpp"

// (the router's arithmetic is spelled out operation by operation: no contraction here)
#pragma clang fp contract(off)

namespace vk {
namespace {

// What route_align_kernel takes: every workgroup routes all the tokens itself, a wavefront
// per token, and keeps the table in LDS.  Up to one token per wavefront (16): a workgroup
// is one compute unit, whose four SIMDs issue the ~300 instructions of a token one
// wavefront instruction per four cycles, so 64 tokens cost it 9 us however the tokens are
// interleaved (measured: 14.2 us for the kernel at 64 tokens and 32 experts, 10.1 us at 32,
// 6.5 us at one, against 4.0 + 5.3 us for the router's own launch, which spreads the tokens
// over the device, followed by the alignment's).
constexpr int kRouteAlignMaxTokens = 16, kRouteAlignMaxRows = 1024, kRouteAlignMaxExperts = 1024;

constexpr int kAlignThreads = 1024;
constexpr int kAlignWaves = kAlignThreads / 64;
constexpr int kAlignAhead = 8;  // chunks of 64 indices a lane has in flight

__device__ __forceinline__ int local_expert(int ge, const int32_t* expert_map,
                                            int num_experts, int local_n) {
  if (ge < 0 || ge >= num_experts) return -1;
  const int le = expert_map ? expert_map[ge] : ge;
  return (le < 0 || le >= local_n) ? -1 : le;
}

__device__ __forceinline__ int block_sum(int v, int* red) {
  // red: kAlignWaves ints of LDS.  Returns the workgroup total to every thread.
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int w = 0; w < kAlignWaves; ++w) t += red[w];
  return t;
}

// The work of workgroup blockIdx.x (steps 1 to 4 above).  topk_ids: the N flat routing
// indices, in global memory or in LDS; hist: local_n ints of LDS.
__device__ __forceinline__ void align_workgroup(
    const int32_t* topk_ids, const int32_t* __restrict__ expert_map,
    int N, int block_size, int num_experts, int local_n, int max_EM,
    int32_t* __restrict__ sorted_ids, int32_t* __restrict__ expert_ids,
    int32_t* __restrict__ out_em, int32_t* hist) {
  __shared__ int wave_cnt[kAlignWaves];
  __shared__ int red[kAlignWaves];

  const int e = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  for (int i = tid; i < local_n; i += kAlignThreads) hist[i] = 0;
  __syncthreads();

  // Slice of the flat indices owned by this wavefront (a multiple of 64 long
  // so that every step of the walk is a full wavefront).
  const int slice = ((N + kAlignWaves - 1) / kAlignWaves + 63) & ~63;
  const int begin = wave * slice;
  const int end = min(N, begin + slice);

  // A lane asks for kAlignAhead chunks of 64 indices before it uses the first: one
  // load per trip makes the walk a chain of round trips to L2 (two walks of N / 1024
  // trips each; N = 131072, 256 experts: 92 us that way, 75 us this way).
  int mine = 0;
  for (int base0 = begin; base0 < end; base0 += 64 * kAlignAhead) {
    int ids_ahead[kAlignAhead];
#pragma unroll
    for (int u = 0; u < kAlignAhead; ++u) ids_ahead[u] = topk_ids[min(base0 + 64 * u + lane, end - 1)];
#pragma unroll
    for (int u = 0; u < kAlignAhead; ++u) {
      const int base = base0 + 64 * u;
      if (base >= end) break;  // uniform
      const int i = base + lane;
      const int le = i < end ? local_expert(ids_ahead[u], expert_map, num_experts, local_n) : -1;
      if (le >= 0) {
        // A wavefront whose lanes all hit one expert adds once instead of
        // serialising 64 atomics on one address.
        const int first = __builtin_amdgcn_readfirstlane(le);
        const unsigned long long same = __ballot(le == first);
        const unsigned long long active = __ballot(1);
        if (same == active) {
          if (lane == (int)__builtin_ctzll(active)) atomicAdd(&hist[first], (int)__popcll(active));
        } else {
          atomicAdd(&hist[le], 1);
        }
      }
      mine += (int)__popcll(__ballot(le == e));
    }
  }
  if (lane == 0) wave_cnt[wave] = mine;
  __syncthreads();

  // Padded rows of the experts before this one, and of all experts.
  int before = 0, total = 0;
  for (int i = tid; i < local_n; i += kAlignThreads) {
    const int c = hist[i];
    const int padded = (c + block_size - 1) / block_size * block_size;
    total += padded;
    if (i < e) before += padded;
  }
  before = block_sum(before, red);
  total = block_sum(total, red);
  int em = total == 0 ? block_size : total;
  if (em > max_EM) em = max_EM;
  if (e == 0 && tid == 0) *out_em = em;

  const int count = e < local_n ? hist[e] : 0;
  const int padded = (count + block_size - 1) / block_size * block_size;

  // Rank of this wavefront's first match among the matches of expert e.
  int wave_base = 0;
  for (int w = 0; w < wave; ++w) wave_base += wave_cnt[w];

  if (count > 0) {
    int running = before + wave_base;
    for (int base0 = begin; base0 < end; base0 += 64 * kAlignAhead) {
      int ids_ahead[kAlignAhead];
#pragma unroll
      for (int u = 0; u < kAlignAhead; ++u) ids_ahead[u] = topk_ids[min(base0 + 64 * u + lane, end - 1)];
#pragma unroll
      for (int u = 0; u < kAlignAhead; ++u) {
        const int base = base0 + 64 * u;
        if (base >= end) break;  // uniform
        const int i = base + lane;
        const int le = i < end ? local_expert(ids_ahead[u], expert_map, num_experts, local_n) : -1;
        const unsigned long long match = __ballot(le == e);
        if (le == e) {
          const int pos = running + (int)__popcll(match & ((1ull << lane) - 1ull));
          if (pos < max_EM) sorted_ids[pos] = i;
        }
        running += (int)__popcll(match);
      }
    }
    for (int r = before + count + tid; r < before + padded; r += kAlignThreads)
      if (r < max_EM) sorted_ids[r] = N;
    const int max_blocks = max_EM / block_size;
    for (int b = before / block_size + tid; b < (before + padded) / block_size; b += kAlignThreads)
      if (b < max_blocks) expert_ids[b] = e;
  }

  // Sentinel tail [total, max_EM): split evenly over the workgroups.
  {
    const int tail0 = min(total, max_EM);
    const int tail = max_EM - tail0;
    const int per = (tail + (int)gridDim.x - 1) / (int)gridDim.x;
    const int lo = tail0 + e * per;
    const int hi = min(max_EM, lo + per);
    for (int r = lo + tid; r < hi; r += kAlignThreads) sorted_ids[r] = N;
    const int b0 = tail0 / block_size, nb = max_EM / block_size - b0;
    const int perb = (nb + (int)gridDim.x - 1) / (int)gridDim.x;
    const int blo = b0 + e * perb;
    const int bhi = min(max_EM / block_size, blo + perb);
    for (int b = blo + tid; b < bhi; b += kAlignThreads) expert_ids[b] = -1;
  }
}

__global__ __launch_bounds__(kAlignThreads) void align_kernel(
    const int32_t* __restrict__ topk_ids, const int32_t* __restrict__ expert_map,
    int N, int block_size, int num_experts, int local_n, int max_EM,
    int32_t* __restrict__ sorted_ids, int32_t* __restrict__ expert_ids,
    int32_t* __restrict__ out_em) {
  extern __shared__ int32_t hist[];  // [local_n]
  align_workgroup(topk_ids, expert_map, N, block_size, num_experts, local_n, max_EM, sorted_ids,
                  expert_ids, out_em, hist);
}

// Router and alignment in one launch, for decode-sized batches: every workgroup routes
// all T tokens itself (a wavefront per token, the same arithmetic as route_topk_kernel,
// so every workgroup holds the same table), keeps the indices in LDS, and then does its
// expert's share of the alignment from there; workgroup 0 also writes the routing
// table out.  One launch less in front of the layer, where a launch is a few
// microseconds of a step of fifty to a hundred.
template <int PER>
__global__ __launch_bounds__(kAlignThreads) void route_align_kernel(
    const float* __restrict__ logits, int T, int E, int top_k, int renormalize,
    const int32_t* __restrict__ expert_map, int block_size, int local_n, int max_EM,
    int32_t* __restrict__ topk_ids, float* __restrict__ topk_w,
    int32_t* __restrict__ sorted_ids, int32_t* __restrict__ expert_ids,
    int32_t* __restrict__ out_em) {
  extern __shared__ int32_t lds[];  // [max(local_n, 1)] histogram, [T * top_k] routing indices
  int32_t* const ids = lds + (local_n > 0 ? local_n : 1);
  const int lane = threadIdx.x & 63;
  for (int token = threadIdx.x >> 6; token < T; token += kAlignWaves) {  // uniform per wavefront
    int my_id;
    float my_w;
    route_token<PER>(logits + (size_t)token * E, E, top_k, renormalize, lane, my_id, my_w);
    if (lane < top_k) {
      ids[token * top_k + lane] = my_id;
      if (blockIdx.x == 0) {
        topk_ids[(size_t)token * top_k + lane] = my_id;
        topk_w[(size_t)token * top_k + lane] = my_w;
      }
    }
  }
  __syncthreads();
  align_workgroup(ids, expert_map, T * top_k, block_size, E, local_n, max_EM, sorted_ids, expert_ids,
                  out_em, lds);
}

}  // namespace

bool route_align_fits(int T, int E, int top_k, int local_n) {
  (void)E;
  return T > 0 && T <= kRouteAlignMaxTokens && top_k <= 64 &&
         (long long)T * top_k <= kRouteAlignMaxRows && local_n <= kRouteAlignMaxExperts;
}

void launch_route_align(const float* logits, int T, int E, int top_k, int renormalize,
                        const int32_t* expert_map, int block_size, int local_n, int max_EM,
                        int32_t* topk_ids, float* topk_w, int32_t* sorted_ids, int32_t* expert_ids,
                        int32_t* out_em, hipStream_t stream) {
  const int groups = local_n > 0 ? local_n : 1;
  const size_t lds = sizeof(int32_t) * ((size_t)groups + (size_t)T * (size_t)top_k);
#define VK_ROUTE_ALIGN_LAUNCH(PER)                                                                     \
  hipLaunchKernelGGL((route_align_kernel<PER>), dim3(groups), dim3(kAlignThreads), lds, stream, logits, \
                     T, E, top_k, renormalize, expert_map, block_size, local_n, max_EM, topk_ids,       \
                     topk_w, sorted_ids, expert_ids, out_em)
  if (E <= 64) VK_ROUTE_ALIGN_LAUNCH(1);
  else if (E <= 128) VK_ROUTE_ALIGN_LAUNCH(2);
  else if (E <= 256) VK_ROUTE_ALIGN_LAUNCH(4);
  else if (E <= 512) VK_ROUTE_ALIGN_LAUNCH(8);
  else VK_ROUTE_ALIGN_LAUNCH(16);
#undef VK_ROUTE_ALIGN_LAUNCH
}

void launch_align(const int32_t* topk_ids, const int32_t* expert_map, int N,
                  int block_size, int num_experts, int local_n, int max_EM,
                  int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_em,
                  hipStream_t stream) {
  // local_n == 0 still needs one workgroup to write the sentinels and EM.
  const int groups = local_n > 0 ? local_n : 1;
  const size_t lds = sizeof(int32_t) * (size_t)(local_n > 0 ? local_n : 1);
  hipLaunchKernelGGL(align_kernel, dim3(groups), dim3(kAlignThreads), lds, stream,
                     topk_ids, expert_map, N, block_size, num_experts, local_n,
                     max_EM, sorted_ids, expert_ids, out_em);
}

}  // namespace vk
