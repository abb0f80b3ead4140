// moe_dequant.hip — device counterpart of dequant_weight_tile
// (src/c/vkernels/kernels/moe_fused.cpp:141-174 of the reference): an [N, K]
// tile of packed E2M1 codes with ue8m0 group scales -> bf16, written
// transposed as [K][N].  It runs the decode routines of mxfp4.hpp, the same
// ones the GEMM kernels use, so that the weight values the GEMMs multiply by
// can be compared bit for bit with the CPU oracle.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxfp4.hpp"
#include "vk_internal.hpp"

namespace vk {
namespace {

// One thread per (row n, group of 8 codes).
__global__ __launch_bounds__(256) void dequant_tile_kernel(
    const uint8_t* __restrict__ packed, const uint8_t* __restrict__ scale,
    uint16_t* __restrict__ out, int N, int K, int stride_packed,
    int stride_scale_n, int stride_scale_k, int fast) {
  const int pieces = K / 8;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)N * pieces) return;
  const int n = (int)(idx / pieces);
  const int piece = (int)(idx % pieces);
  const uint8_t* src = packed + (size_t)n * stride_packed + (size_t)piece * 4;
  const uint32_t x = (uint32_t)src[0] | ((uint32_t)src[1] << 8) |
                     ((uint32_t)src[2] << 16) | ((uint32_t)src[3] << 24);
  const uint32_t s = scale[(size_t)n * stride_scale_n + (size_t)(piece / 4) * stride_scale_k];
  const u32x4 v = fast ? dequant8_fast(x, scale_half_f32(s)) : dequant8_exact(x, s);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = piece * 8 + 2 * i;
    out[(size_t)k * N + n] = (uint16_t)(v[i] & 0xFFFFu);
    out[(size_t)(k + 1) * N + n] = (uint16_t)(v[i] >> 16);
  }
}

}  // namespace

void launch_dequant_tile(const uint8_t* packed, const uint8_t* scale,
                         uint16_t* out_bf16, int N, int K, int stride_packed,
                         int stride_scale_n, int stride_scale_k, int fast,
                         hipStream_t stream) {
  const long long total = (long long)N * (K / 8);
  if (total <= 0) return;
  const int threads = 256;
  const unsigned blocks = (unsigned)((total + threads - 1) / threads);
  hipLaunchKernelGGL(dequant_tile_kernel, dim3(blocks), dim3(threads), 0, stream,
                     packed, scale, out_bf16, N, K, stride_packed, stride_scale_n,
                     stride_scale_k, fast);
}

}  // namespace vk
