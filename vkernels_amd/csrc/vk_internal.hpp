// vk_internal.hpp — launchers shared between the kernel translation units and
// the C ABI.  Not part of the public interface.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vk {

void launch_route_topk(const float* logits, int T, int E, int top_k,
                       int renormalize, int32_t* topk_ids, float* topk_w,
                       hipStream_t stream);

void launch_align(const int32_t* topk_ids, const int32_t* expert_map, int N,
                  int block_size, int num_experts, int local_n, int max_EM,
                  int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_em,
                  hipStream_t stream);

void launch_dequant_tile(const uint8_t* packed, const uint8_t* scale,
                         uint16_t* out_bf16, int N, int K, int stride_packed,
                         int stride_scale_n, int stride_scale_k, int fast,
                         hipStream_t stream);

struct FusedMoeArgs {
  const uint16_t* A;
  const uint8_t* w13;
  const uint8_t* w13_scale;
  const uint8_t* w2;
  const uint8_t* w2_scale;
  const float* topk_w;
  uint16_t* act;
  float* out;
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const float* b13;
  const float* b2;
  int M, hidden, ispp, top_k, EM, block_size;
  float swiglu_limit, beta, linear_beta;
  int activation;
  void* workspace;         // optional, see fused_moe_workspace_bytes
  size_t workspace_bytes;
  unsigned flags;          // VK_HIP_MOE_* of vkernels_hip.h
};

// Bytes of workspace with which launch_fused_moe runs its fastest path.
size_t fused_moe_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM);

void launch_fused_moe(const FusedMoeArgs& a, hipStream_t stream);
void launch_moe_gateup(const FusedMoeArgs& a, hipStream_t stream);
void launch_moe_down(const FusedMoeArgs& a, hipStream_t stream);

// Per-kernel set-up that the launchers otherwise do on their first call (the
// dynamic-LDS limits of the GEMM kernels), for callers that want it done before
// a graph capture.  False when the device refuses a limit.
bool prepare_moe_kernels();

// The library-held workspace of vk_hip_fused_moe_mxfp4_static
// (static_scratch.hip): its size, and the address of the current device's copy.
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
size_t static_scratch_bytes();
void* static_scratch_ptr(hipError_t* err);

}  // namespace vk
