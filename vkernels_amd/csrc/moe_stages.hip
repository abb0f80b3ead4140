// moe_stages.hip — the elementwise stages of the layer as kernels of their own: the
// activation epilogue on fp32 pre-activations and the routed combine in gather form.
//
// They are what a tensor-parallel caller runs between its all-reduces (the reference's
// stage split, src/c/vkernels/kernels/moe_fused.hpp:103-125 and :259-283: gate/up GEMM ->
// all-reduce -> activation epilogue -> down GEMM -> all-reduce -> combine), and the
// combine is also the device form of mxfp4_moe_scatter_reduce
// (src/c/vkernels/kernels/moe_aux.cpp:265-285).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "moe_common.hpp"
#include "vk_internal.hpp"

namespace vk {
namespace {

// act[r, c] = bf16(activation(gate_up[r, c] + b13[e, c], gate_up[r, ispp + c] + b13[e, ispp + c]))
// for every routed sorted row r of a block with an expert (moe_act_epilogue_cpu,
// src/c/vkernels/kernels/moe_fused.cpp:370-422); the other rows of act are left as they
// are.  One thread per 4 columns.
__global__ __launch_bounds__(256) void act_epilogue_kernel(
    const float* __restrict__ gate_up, const float* __restrict__ b13, uint16_t* __restrict__ act,
    const int32_t* __restrict__ sorted_ids, const int32_t* __restrict__ expert_ids, int n_flat, int EM,
    int ispp, int block_size, float swiglu_limit, int activation, float beta, float linear_beta) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= ispp) return;
  for (int r = blockIdx.y; r < EM; r += gridDim.y) {
    const int flat = sorted_ids[r];
    const int e = expert_ids[r / block_size];
    if (flat < 0 || flat >= n_flat || e < 0) continue;
    const float* row = gate_up + (size_t)r * (size_t)(2 * ispp);
    f32x4 g = *reinterpret_cast<const f32x4*>(row + c);
    f32x4 u = *reinterpret_cast<const f32x4*>(row + ispp + c);
    if (b13 != nullptr) {
      const float* b = b13 + (size_t)e * (size_t)(2 * ispp);
      g += *reinterpret_cast<const f32x4u*>(b + c);
      u += *reinterpret_cast<const f32x4u*>(b + ispp + c);
    }
    uint32_t v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[i] = f32_to_bf16_bits(act_value(activation, g[i], u[i], swiglu_limit, beta, linear_beta));
    *reinterpret_cast<uint2*>(act + (size_t)r * (size_t)ispp + c) =
        make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
  }
}

// pos[flat] = sorted row of every routed flat index (the others keep their -1).
__global__ __launch_bounds__(256) void invert_sorted_ids_kernel(const int32_t* __restrict__ sorted_ids,
                                                                int32_t* __restrict__ pos, int EM,
                                                                int n_flat) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= EM) return;
  const int flat = sorted_ids[r];
  if (flat >= 0 && flat < n_flat) pos[flat] = r;
}

// Routed combine in gather form: out[t, :] += (partial[r, :] + bias[e(r), :]) * w[r] over
// the token's sorted rows r in ascending order, which is the order the reference's loops
// over the rows add them in (moe_combine_cpu, moe_fused.cpp:523-564; without a bias,
// mxfp4_moe_scatter_reduce, moe_aux.cpp:265-285).  The sum with the bias, the product and
// the sum into out are each rounded on their own, as there, so the result is the
// reference's bit for bit.  A row of a block without an expert (expert_ids given) adds
// nothing.  One thread per 4 columns.
__global__ __launch_bounds__(256) void combine_rows_kernel(
    const float* __restrict__ partial, const float* __restrict__ bias, const float* __restrict__ w_sorted,
    const int32_t* __restrict__ pos, const int32_t* __restrict__ expert_ids, float* __restrict__ out,
    int M, int width, int top_k, int block_size) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= width) return;
  for (int t = blockIdx.y; t < M; t += gridDim.y) {
    f32x4u* o = reinterpret_cast<f32x4u*>(out + (size_t)t * (size_t)width + c);
    f32x4 sum = *o;
    int last = -1;
    for (int s = 0; s < top_k; ++s) {   // the next larger sorted row of this token (top_k is small)
      int r = 0x7FFFFFFF;
      for (int j = 0; j < top_k; ++j) {
        const int rj = pos[t * top_k + j];
        if (rj > last && rj < r) r = rj;
      }
      if (r == 0x7FFFFFFF) break;
      last = r;
      int e = 0;
      if (expert_ids != nullptr) e = expert_ids[r / block_size];
      if (e < 0) continue;
      f32x4 p = *reinterpret_cast<const f32x4u*>(partial + (size_t)r * (size_t)width + c);
      if (bias != nullptr) p += *reinterpret_cast<const f32x4u*>(bias + (size_t)e * (size_t)width + c);
      const float w = w_sorted[r];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float prod = p[i] * w;
        asm volatile("" : "+v"(prod));   // the rounded product is a value of its own: no fused multiply-add
        sum[i] += prod;
      }
    }
    *o = sum;
  }
}

// dst[r, :] = src[sorted_ids[r] / top_k, :] for every sorted row r, rows of row_bytes
// bytes; a padding row (id outside [0, n_flat)) is zeroed (mxfp4_moe_sort and
// mxfp4_moe_sort_scales, src/c/vkernels/kernels/moe_aux.cpp:209-260).  One workgroup per
// sorted row.  VEC: rows and bases are multiples of 16 bytes.
template <bool VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint8_t* __restrict__ src,
                                                          const int32_t* __restrict__ sorted_ids,
                                                          uint8_t* __restrict__ dst, size_t row_bytes,
                                                          int top_k, int n_flat) {
  const size_t r = blockIdx.x;
  const int flat = sorted_ids[r];
  const bool pad = flat < 0 || flat >= n_flat;
  const uint8_t* from = src + (size_t)(pad ? 0 : flat / top_k) * row_bytes;
  uint8_t* to = dst + r * row_bytes;
  if (VEC) {
    for (size_t i = (size_t)threadIdx.x * 16; i < row_bytes; i += 256 * 16) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (!pad) v = *reinterpret_cast<const u32x4*>(from + i);
      *reinterpret_cast<u32x4*>(to + i) = v;
    }
  } else {
    for (size_t i = threadIdx.x; i < row_bytes; i += 256) to[i] = pad ? (uint8_t)0 : from[i];
  }
}

// The routed combine of a quantised partial (mxfp4_moe_scatter_reduce_q, moe_aux.cpp:288-321):
// out[t, c] += (value(code[r, c]) * 2^(s[r, c / 32] - 127)) * w[r] over the token's sorted
// rows r in ascending order, a scale byte of 0xFF standing for zero and one of 0 for +0.0
// (moe_aux.cpp:76-82: the bits s << 23).  The dequantised value, its product with the
// routing weight and the sum into out are each rounded on their own, as there.  Gather
// form over the table of sorted positions; one thread per 8 columns (4 bytes of codes).
__global__ __launch_bounds__(256) void combine_rows_q_kernel(
    const uint8_t* __restrict__ partial_q, const uint8_t* __restrict__ partial_s,
    const float* __restrict__ w_sorted, const int32_t* __restrict__ pos, float* __restrict__ out, int M,
    int width, int top_k) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= width) return;
  const int groups = width / 32;
  for (int t = blockIdx.y; t < M; t += gridDim.y) {
    float* o = out + (size_t)t * (size_t)width + c;
    float sum[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sum[i] = o[i];
    int last = -1;
    for (int s = 0; s < top_k; ++s) {   // the next larger sorted row of this token (top_k is small)
      int r = 0x7FFFFFFF;
      for (int j = 0; j < top_k; ++j) {
        const int rj = pos[t * top_k + j];
        if (rj > last && rj < r) r = rj;
      }
      if (r == 0x7FFFFFFF) break;
      last = r;
      const uint32_t codes = *reinterpret_cast<const uint32_t*>(partial_q + (size_t)r * (size_t)(width / 2) + c / 2);
      const uint32_t sb = partial_s[(size_t)r * (size_t)groups + c / 32];
      const float scale = sb == 0xFFu ? 0.0f : __uint_as_float(sb << 23);
      const float w = w_sorted[r];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float v = __uint_as_float(fp4nib_to_f32bits((codes >> (4 * i)) & 15u)) * scale;
        asm volatile("" : "+v"(v));      // each product is a rounded value of its own: nothing is fused
        float prod = v * w;
        asm volatile("" : "+v"(prod));
        sum[i] += prod;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = sum[i];
  }
}

}  // namespace

void launch_mxfp4_gather_rows(const void* src, const int32_t* sorted_ids, void* dst, size_t row_bytes,
                              int top_k, int n_flat, int EM, hipStream_t stream) {
  if (EM <= 0 || row_bytes == 0) return;
  const bool vec = row_bytes % 16 == 0 &&
                   ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
  if (vec)
    hipLaunchKernelGGL(gather_rows_kernel<true>, dim3((unsigned)EM), dim3(256), 0, stream,
                       static_cast<const uint8_t*>(src), sorted_ids, static_cast<uint8_t*>(dst), row_bytes,
                       top_k, n_flat);
  else
    hipLaunchKernelGGL(gather_rows_kernel<false>, dim3((unsigned)EM), dim3(256), 0, stream,
                       static_cast<const uint8_t*>(src), sorted_ids, static_cast<uint8_t*>(dst), row_bytes,
                       top_k, n_flat);
}

void launch_mxfp4_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s, const float* topk_w,
                                   const int32_t* sorted_ids, float* out, int M, int width, int top_k,
                                   int EM, int32_t* pos, hipStream_t stream) {
  if (M <= 0 || width <= 0 || EM <= 0) return;
  launch_fill_i32(pos, -1, M * top_k, stream);
  hipLaunchKernelGGL(invert_sorted_ids_kernel, dim3((unsigned)((EM + 255) / 256)), dim3(256), 0, stream,
                     sorted_ids, pos, EM, M * top_k);
  const dim3 grid((unsigned)((width / 8 + 255) / 256), (unsigned)(M < 65535 ? M : 65535));
  hipLaunchKernelGGL(combine_rows_q_kernel, grid, dim3(256), 0, stream, partial_q, partial_s, topk_w, pos,
                     out, M, width, top_k);
}

void launch_moe_act_epilogue(const float* gate_up, const float* b13, uint16_t* act,
                             const int32_t* sorted_ids, const int32_t* expert_ids, int M, int top_k, int EM,
                             int ispp, int block_size, float swiglu_limit, int activation, float beta,
                             float linear_beta, hipStream_t stream) {
  if (M <= 0 || EM <= 0 || ispp <= 0) return;
  const dim3 grid((unsigned)((ispp / 4 + 255) / 256), (unsigned)(EM < 65535 ? EM : 65535));
  hipLaunchKernelGGL(act_epilogue_kernel, grid, dim3(256), 0, stream, gate_up, b13, act, sorted_ids,
                     expert_ids, M * top_k, EM, ispp, block_size, swiglu_limit, activation, beta,
                     linear_beta);
}

void launch_moe_combine_sorted(const float* partial, const float* bias, const float* w_sorted,
                               const int32_t* sorted_ids, const int32_t* expert_ids, float* out, int M,
                               int width, int top_k, int EM, int block_size, int32_t* pos,
                               hipStream_t stream) {
  if (M <= 0 || width <= 0 || EM <= 0) return;
  launch_fill_i32(pos, -1, M * top_k, stream);
  hipLaunchKernelGGL(invert_sorted_ids_kernel, dim3((unsigned)((EM + 255) / 256)), dim3(256), 0, stream,
                     sorted_ids, pos, EM, M * top_k);
  const dim3 grid((unsigned)((width / 4 + 255) / 256), (unsigned)(M < 65535 ? M : 65535));
  hipLaunchKernelGGL(combine_rows_kernel, grid, dim3(256), 0, stream, partial, bias, w_sorted, pos,
                     expert_ids, out, M, width, top_k, block_size > 0 ? block_size : 16);
}

void launch_mxfp4_scatter_reduce(const float* partial, const float* topk_w, const int32_t* sorted_ids,
                                 float* out, int M, int width, int top_k, int EM, int32_t* pos,
                                 hipStream_t stream) {
  launch_moe_combine_sorted(partial, nullptr, topk_w, sorted_ids, nullptr, out, M, width, top_k, EM, 16, pos,
                            stream);
}

}  // namespace vk
