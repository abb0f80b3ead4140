// ref_shim.cpp — extern "C" doorway into a build of the reference's own
// moe_fused.cpp.  TEST INFRASTRUCTURE ONLY.
//
// Compiled (by oracle/Makefile, target `ref`) together with
// /root/reference/src/c/vkernels/kernels/moe_fused.cpp, straight from where
// that file lies, into oracle/_ref/libvkref.so.  Used to check the oracle's
// restatement bit for bit and as the reference CPU baseline of the benchmark.
// No reference source is copied into this repository.
#include <cstddef>
#include <cstdint>

#include "vkernels/kernels/moe_aux.hpp"
#include "vkernels/kernels/moe_fused.hpp"

namespace vk = vkernels::kernels;

extern "C" {

void vkref_fused_moe_mxfp4(const uint16_t* A, const uint8_t* w13,
                           const uint8_t* w13_scale, const uint8_t* w2,
                           const uint8_t* w2_scale, const int32_t* sorted_ids,
                           const float* topk_w_sorted,
                           const int32_t* expert_ids, uint16_t* act_scratch,
                           float* out, int M, int hidden, int ispp, int top_k,
                           int EM, int group_size, float swiglu_limit,
                           int activation, float beta, float linear_beta,
                           const float* b13, const float* b2) {
  vk::fused_moe_mxfp4_cpu(A, w13, w13_scale, w2, w2_scale, sorted_ids,
                          topk_w_sorted, expert_ids, act_scratch, out, M,
                          hidden, ispp, top_k, EM, group_size, swiglu_limit,
                          activation, beta, linear_beta, b13, b2);
}

void vkref_moe_gateup(const uint16_t* A, const uint8_t* w13,
                      const uint8_t* w13_scale, const int32_t* sorted_ids,
                      const int32_t* expert_ids, float* gate_up, int M,
                      int a_stride, int k_base, int hidden_k, int ispp,
                      int top_k, int EM, int group_size) {
  vk::moe_gateup_cpu(A, w13, w13_scale, sorted_ids, expert_ids, gate_up, M,
                     a_stride, k_base, hidden_k, ispp, top_k, EM, group_size);
}

void vkref_moe_act_epilogue(const float* gate_up, const float* b13,
                            uint16_t* act, const int32_t* sorted_ids,
                            const int32_t* expert_ids, int M, int top_k,
                            int EM, int ispp, float swiglu_limit,
                            int activation, float beta, float linear_beta) {
  vk::moe_act_epilogue_cpu(gate_up, b13, act, sorted_ids, expert_ids, M, top_k,
                           EM, ispp, swiglu_limit, activation, beta,
                           linear_beta);
}

void vkref_moe_down(const uint16_t* act, const uint8_t* w2,
                    const uint8_t* w2_scale, const int32_t* sorted_ids,
                    const int32_t* expert_ids, float* partial, int M,
                    int a_stride, int k_base, int ispp_k, int hidden,
                    int top_k, int EM, int group_size) {
  vk::moe_down_cpu(act, w2, w2_scale, sorted_ids, expert_ids, partial, M,
                   a_stride, k_base, ispp_k, hidden, top_k, EM, group_size);
}

void vkref_moe_combine(const float* partial, const float* b2,
                       const float* topk_w_sorted, const int32_t* sorted_ids,
                       const int32_t* expert_ids, float* out, int M,
                       int hidden, int top_k, int EM) {
  vk::moe_combine_cpu(partial, b2, topk_w_sorted, sorted_ids, expert_ids, out,
                      M, hidden, top_k, EM);
}

int vkref_moe_align_block_size(const int32_t* topk_ids, int M, int top_k,
                               int block_size, int num_experts,
                               int32_t* sorted_ids, int32_t* expert_ids) {
  return vk::moe_align_block_size(topk_ids, M, top_k, block_size, num_experts,
                                  sorted_ids, expert_ids);
}

void vkref_dequant_weight_tile(const uint8_t* packed, const uint8_t* scale,
                               uint16_t* out_bf16, int N, int K,
                               int group_size, int stride_packed,
                               int stride_scale_n, int stride_scale_k) {
  vk::dequant_weight_tile(packed, scale, out_bf16, N, K, group_size,
                          stride_packed, stride_scale_n, stride_scale_k);
}

void vkref_dequant_weight_tile_ref(const uint8_t* packed, const uint8_t* scale,
                                   uint16_t* out_bf16, int N, int K,
                                   int group_size, int stride_packed,
                                   int stride_scale_n, int stride_scale_k) {
  vk::dequant_weight_tile_ref(packed, scale, out_bf16, N, K, group_size,
                              stride_packed, stride_scale_n, stride_scale_k);
}


// ---- moe_aux.cpp ----
void vkref_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int M, int hidden,
                           int group_size) {
  vk::mxfp4_moe_quant(A, packed, scales, M, hidden, group_size);
}

void vkref_mxfp4_moe_sorted_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed,
                                  uint8_t* scales, int M, int hidden, int group_size, int top_k,
                                  int EM) {
  vk::mxfp4_moe_sorted_quant(A, sorted_ids, packed, scales, M, hidden, group_size, top_k, EM);
}

void vkref_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int M,
                          int hidden, int top_k, int EM) {
  vk::mxfp4_moe_sort(A, sorted_ids, A_sorted, M, hidden, top_k, EM);
}

void vkref_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids,
                                 uint8_t* scales_sorted, int M, int n_groups, int top_k, int EM) {
  vk::mxfp4_moe_sort_scales(scales, sorted_ids, scales_sorted, M, n_groups, top_k, EM);
}

void vkref_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w,
                                    const int32_t* sorted_ids, float* out, int M, int width,
                                    int top_k, int EM) {
  vk::mxfp4_moe_scatter_reduce(partial, topk_w, sorted_ids, out, M, width, top_k, EM);
}

void vkref_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                      const float* topk_w, const int32_t* sorted_ids, float* out,
                                      int M, int width, int top_k, int EM, int group_size) {
  vk::mxfp4_moe_scatter_reduce_q(partial_q, partial_s, topk_w, sorted_ids, out, M, width, top_k,
                                 EM, group_size);
}

}  // extern "C"
