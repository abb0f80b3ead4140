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

// Router and alignment of a decode-sized batch in one launch (route_align_fits says
// whether the shape is one it takes).
bool route_align_fits(int T, int E, int top_k, int local_n);
void launch_route_align(const float* logits, int T, int E, int top_k, int renormalize,
                        const int32_t* expert_map, int block_size, int local_n, int max_EM,
                        int32_t* topk_ids, float* topk_w, int32_t* sorted_ids, int32_t* expert_ids,
                        int32_t* out_em, hipStream_t stream);

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
  // optional: the weights prepacked by launch_moe_prepack (both or neither)
  const uint8_t* w13_packed;
  const uint8_t* w2_packed;
  int num_experts;         // experts in the weight tensors (needed with prepacked weights)
};

// Bytes of workspace with which launch_fused_moe runs its fastest path.
size_t fused_moe_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM);

void launch_fused_moe(const FusedMoeArgs& a, hipStream_t stream);

// Router + alignment + layer in one call (vk_hip_moe_route_layer_mxfp4): what the router
// and the alignment read and write besides the layer's own arguments.
struct RoutedArgs {
  const float* logits;        // [M, num_experts]
  const int32_t* expert_map;  // or null
  int32_t* topk_ids;          // [M, top_k] out
  float* topk_w;              // [M, top_k] out
  int32_t* sorted_ids;        // [max_EM] out
  int32_t* expert_ids;        // [max_EM / block_size] out
  int32_t* out_EM;            // out
  int num_experts, local_n, renormalize, max_EM;
};
// The two-launch form for a handful of tokens; false (nothing enqueued) when the call
// is not one it takes.
bool launch_routed_moe(const FusedMoeArgs& a, const RoutedArgs& r, hipStream_t stream);
void launch_moe_gateup(const FusedMoeArgs& a, hipStream_t stream);
void launch_moe_down(const FusedMoeArgs& a, hipStream_t stream);

// Pieces of the workspace path shared between the translation units.
void launch_fill_i32(int32_t* dst, int32_t value, int n, hipStream_t stream);
void launch_combine(const float* y, const int32_t* pos, float* out, int M, int top_k, int hidden,
                    bool overwrite, hipStream_t stream);

// Prepacked weights (moe_prefill.hip): bytes of the packed form of [num_experts, rows,
// K/2] codes + [num_experts, rows, K/32] scales (stage 0: rows = 2 * ispp, gate rows
// first; stage 1: rows = hidden), the packing launch, and the layer on packed weights.
size_t moe_prepack_bytes(int num_experts, int rows, int K, int stage);
void launch_moe_prepack(const uint8_t* w, const uint8_t* w_scale, int num_experts, int rows, int K,
                        int stage, uint8_t* packed, hipStream_t stream);
size_t mx_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM);
bool launch_fused_moe_prepacked(const FusedMoeArgs& a, hipStream_t stream);
bool fused_moe_prepacked_takes(const FusedMoeArgs& a, bool both_stages);
// A call with the prepacked weights alone (w13 / w2 null): can the library run it?
// (the layer; the second stage alone)
bool fused_moe_packed_only_ok(const FusedMoeArgs& a);
bool moe_gateup_packed_only_ok(const FusedMoeArgs& a);  // (decode sizes only)
bool moe_down_packed_only_ok(const FusedMoeArgs& a);
bool launch_moe_down_prepacked(const FusedMoeArgs& a, hipStream_t stream);
void launch_split_rows_fp6(const uint16_t* x, int rows, int K, int terms, uint8_t* xq, uint8_t* row_bad,
                           hipStream_t stream);
bool prepare_mx_kernels();

// MXFP4 orchestration ops (moe_prefill.hip): activation quantisation in the ABI layout
// (sorted_ids null = token order), routed combine in gather form (pos: M * top_k ints).
void launch_mxfp4_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed, uint8_t* scales,
                        int rows, int hidden, int top_k, int n_flat, hipStream_t stream);
bool launch_moe_preact(int stage, const uint16_t* a, const uint8_t* w, const uint8_t* w_scale,
                       const int32_t* sorted_ids, const int32_t* expert_ids, float* preact, int M,
                       int a_stride, int ncols, int top_k, int EM, int k_base, int k_dim, int block_size,
                       hipStream_t stream, const uint8_t* packed = nullptr, int num_experts = 0);
// The same on prepacked weights (the FP4-rate kernels of moe_prefill.hip; `packed` from
// launch_moe_prepack for the shard [num_experts, rows, k_dim / 2]); false = nothing enqueued.
size_t mx_preact_workspace_bytes(int stage, int M, int EM, int k_dim);
bool launch_moe_preact_prepacked(int stage, const uint16_t* a, const uint8_t* packed, const uint8_t* w,
                                 const uint8_t* w_scale, const int32_t* sorted_ids, const int32_t* expert_ids,
                                 float* preact, int M, int a_stride, int ncols, int top_k, int EM, int k_base,
                                 int k_dim, int block_size, int num_experts, void* workspace,
                                 size_t workspace_bytes, unsigned flags, hipStream_t stream);
void launch_moe_act_epilogue(const float* gate_up, const float* b13, uint16_t* act,
                             const int32_t* sorted_ids, const int32_t* expert_ids, int M, int top_k, int EM,
                             int ispp, int block_size, float swiglu_limit, int activation, float beta,
                             float linear_beta, hipStream_t stream);
void launch_moe_combine_sorted(const float* partial, const float* bias, const float* w_sorted,
                               const int32_t* sorted_ids, const int32_t* expert_ids, float* out, int M,
                               int width, int top_k, int EM, int block_size, int32_t* pos,
                               hipStream_t stream);
void launch_mxfp4_scatter_reduce(const float* partial, const float* topk_w, const int32_t* sorted_ids,
                                 float* out, int M, int width, int top_k, int EM, int32_t* pos,
                                 hipStream_t stream);

// Rows gathered into sorted order (mxfp4_moe_sort / _sort_scales: rows of row_bytes bytes,
// padding rows zeroed) and the routed combine of a quantised partial (pos: M * top_k ints).
void launch_mxfp4_gather_rows(const void* src, const int32_t* sorted_ids, void* dst, size_t row_bytes,
                              int top_k, int n_flat, int EM, hipStream_t stream);
void launch_mxfp4_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s, const float* topk_w,
                                   const int32_t* sorted_ids, float* out, int M, int width, int top_k,
                                   int EM, int32_t* pos, hipStream_t stream);

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
