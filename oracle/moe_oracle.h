/*
 * moe_oracle.h — CPU restatement of the reference's fused MXFP4 MoE path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped GPU path includes, links
 * or calls this code; it exists so that tests, the smoke check and the CPU
 * leg of the benchmark have an independent checker to compare the HIP
 * kernels against.
 *
 * Every function restates one function of the reference
 * (src/c/vkernels/kernels/moe_fused.cpp and friends); the file:line it
 * follows is cited at each declaration.  Results are bit-identical to the
 * reference for every function that has a reference counterpart (checked by
 * tests/test_oracle_vs_ref.py against a build of the reference translation
 * unit, and frozen in tests/golden/).  vko_route_topk has no counterpart in
 * the reference's CPU code: it is pinned by closed forms, brute force and
 * the softmax/top-k of an independent library.
 *
 * Parity status: every function below is pinned (none is "parity unpinned").
 */
#ifndef VKERNELS_AMD_ORACLE_MOE_ORACLE_H_
#define VKERNELS_AMD_ORACLE_MOE_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { VKO_SWIGLU = 0, VKO_SITU = 1 };

/* E2M1 nibble -> fp32 bit pattern.  Follows moe_fused.cpp:24-39: codes
 * decode to {0, .25, 1, 1.5, 2, 3, inf, NaN} with the sign in bit 3. */
uint32_t vko_fp4nib_to_f32bits(int nibble);

/* ue8m0 scale byte -> float.  Follows moe_fused.cpp:50-64: 0xFF -> 0.0,
 * 1..254 -> 2^(s-127), 0 -> 2^-127 (a subnormal). */
float vko_ue8m0_to_float(uint8_t s);

/* fp32 bits -> bf16, round-to-nearest-even by the +0x7FFF+lsb trick with no
 * NaN special case.  Follows moe_fused.cpp:41-45. */
uint16_t vko_f32bits_to_bf16(uint32_t bits);

/* Dequantise an [N,K] tile of packed weights to bf16, transposed to [K][N].
 * Follows moe_fused.cpp:141-174 (table-driven) and :183-201 (per byte). */
void vko_dequant_weight_tile(const uint8_t* packed, const uint8_t* scale,
                             uint16_t* out_bf16, int N, int K, int group_size,
                             int stride_packed, int stride_scale_n,
                             int stride_scale_k);
void vko_dequant_weight_tile_ref(const uint8_t* packed, const uint8_t* scale,
                                 uint16_t* out_bf16, int N, int K,
                                 int group_size, int stride_packed,
                                 int stride_scale_n, int stride_scale_k);

/* SwiGLU / SiTU epilogue of one (gate, up) pair.  moe_fused.cpp:206-226. */
float vko_epilogue_value(int activation, float g, float u, float swiglu_limit,
                         float beta, float linear_beta);

/* Stage 0a: gate_up[EM, 2*ispp] = A_sorted @ w13^T.  moe_fused.cpp:235-365. */
void vko_moe_gateup(const uint16_t* A, const uint8_t* w13,
                    const uint8_t* w13_scale, const int32_t* sorted_ids,
                    const int32_t* expert_ids, float* gate_up, int M,
                    int a_stride, int k_base, int hidden_k, int ispp,
                    int top_k, int EM, int group_size);

/* Stage 0b: act[EM, ispp] = bf16(act(gate_up + b13)).  moe_fused.cpp:370-422. */
void vko_moe_act_epilogue(const float* gate_up, const float* b13,
                          uint16_t* act, const int32_t* sorted_ids,
                          const int32_t* expert_ids, int M, int top_k, int EM,
                          int ispp, float swiglu_limit, int activation,
                          float beta, float linear_beta);

/* Stage 1a: partial[EM, hidden] = act @ w2^T.  moe_fused.cpp:427-518. */
void vko_moe_down(const uint16_t* act, const uint8_t* w2,
                  const uint8_t* w2_scale, const int32_t* sorted_ids,
                  const int32_t* expert_ids, float* partial, int M,
                  int a_stride, int k_base, int ispp_k, int hidden, int top_k,
                  int EM, int group_size);

/* Stage 1b: out[M, hidden] += (partial + b2) * topk_w_sorted.
 * moe_fused.cpp:523-564. */
void vko_moe_combine(const float* partial, const float* b2,
                     const float* topk_w_sorted, const int32_t* sorted_ids,
                     const int32_t* expert_ids, float* out, int M, int hidden,
                     int top_k, int EM);

/* The four stages composed.  moe_fused.cpp:569-603. */
void vko_fused_moe_mxfp4(const uint16_t* A, const uint8_t* w13,
                         const uint8_t* w13_scale, const uint8_t* w2,
                         const uint8_t* w2_scale, const int32_t* sorted_ids,
                         const float* topk_w_sorted, const int32_t* expert_ids,
                         uint16_t* act_scratch, float* out, int M, int hidden,
                         int ispp, int top_k, int EM, int group_size,
                         float swiglu_limit, int activation, float beta,
                         float linear_beta, const float* b13, const float* b2);

/* Routing table -> block-aligned sorted layout; returns EM (0 when nothing
 * routes).  moe_fused.cpp:609-661. */
int vko_moe_align_block_size(const int32_t* topk_ids, int M, int top_k,
                             int block_size, int num_experts,
                             int32_t* sorted_ids, int32_t* expert_ids);

/* The expert_map-aware variant the serving binding and the device kernel
 * implement: global->local remap, ids outside [0,num_experts) or mapped
 * outside [0,local_n) skipped, EM at least one block, and ALL max_EM /
 * max_EM/block_size output entries written (sentinels N and -1).  Follows
 * src/python/vkernels/vllm_experts.py:297-372 and
 * src/c/vkernels/kernels/moe_fused.hip:1983-2071. */
int vko_moe_align_block_size_with_map(const int32_t* topk_ids,
                                      const int32_t* expert_map, int N,
                                      int block_size, int num_experts,
                                      int local_n, int max_EM,
                                      int32_t* sorted_ids,
                                      int32_t* expert_ids);

/* (ceil(N/bs)+E)*bs.  capi/capi_moe.cpp:110-117. */
size_t vko_align_max_em(int M, int top_k, int block_size, int num_experts);

/* Host upper bound on EM used by the serving path.
 * src/python/vkernels/vllm_experts.py:481-500. */
int vko_align_em_bound(int M, int top_k, int local_n, int block_size);

/* Softmax -> top-k (ties to the lowest expert index) -> optional
 * renormalisation.  Semantics from
 * src/python/vkernels/torch_ops/tokenspeed_amd/routing.py:59-157 (no bias,
 * scaling factor 1).  The arithmetic is fully specified (see router_oracle.c)
 * so that a device implementation can match it bit for bit. */
void vko_route_topk(const float* logits, int T, int E, int top_k,
                    int renormalize, int32_t* topk_ids, float* topk_w);

/* The deterministic exp(x), x <= 0, used by vko_route_topk. */
float vko_route_exp(float x);

/* Number of OpenMP threads the GEMM stages use (1 = the reference's own
 * single-threaded behaviour; results are identical for any value). */
void vko_set_threads(int n);

/* Not in the reference: terms = 2 or 3: the grouped GEMMs multiply the sum of
 * that many FP6 (E2M3) terms per activation block of 32 that the GPU's prefill
 * kernels use; 0 (default) = the reference's arithmetic. */
void vko_set_act_model(int terms);
void vko_act_model_block32(const uint16_t* a, float* out, int terms);

/* ---- MXFP4 MoE orchestration ops (aux_oracle.c; moe_aux.cpp of the reference) ---- */
uint8_t vko_aux_scale_byte(uint16_t amax_bits);
void vko_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int M, int hidden,
                         int group_size);
void vko_mxfp4_moe_sorted_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed,
                                uint8_t* scales, int M, int hidden, int group_size, int top_k,
                                int EM);
void vko_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int M,
                        int hidden, int top_k, int EM);
void vko_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids,
                               uint8_t* scales_sorted, int M, int n_groups, int top_k, int EM);
void vko_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w,
                                  const int32_t* sorted_ids, float* out, int M, int width,
                                  int top_k, int EM);
void vko_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                    const float* topk_w, const int32_t* sorted_ids, float* out,
                                    int M, int width, int top_k, int EM, int group_size);
/* Not in the reference: the values a W4A4 layer multiplies for one group of 32 bf16
 * activations (quantised as mxfp4_moe_quant does, then dequantised). */
void vko_aux_model_block32(const uint16_t* a, float* out);

#ifdef __cplusplus
}
#endif
#endif
