/*
 * vkernels_cpu.h — the host-side (CPU) C ABI of the fused MXFP4 MoE path.
 *
 * These are the reference's own CPU entry points for the path
 * (src/c/vkernels/capi/capi.hpp:470-539, implemented in
 * src/c/vkernels/capi/capi_moe.cpp:20-140): the scalar oracle of the layer,
 * the alignment, and the MXFP4 orchestration ops.  In this repository they are
 * served by the CPU checker only (oracle/liboracle.so, test infrastructure):
 * the product is the device library declared in vkernels_hip.h, and nothing in
 * it falls back to these.  The header exists so that a C or FFI consumer
 * written against the reference's host library (its Rust crate, its C tests)
 * can be compiled and linked against the checker unchanged, and so that the
 * checker's signatures are held to the reference's by a compiler.
 *
 * Conventions (capi.hpp:41-71): every function returns VK_OK or a VK_ERROR_*
 * code and leaves a message for vk_last_error() on failure; plain pointers and
 * sizes, caller-owned host buffers, no allocation.
 */
#ifndef VKERNELS_CPU_H_
#define VKERNELS_CPU_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef VKERNELS_STATUS_CODES_
#define VKERNELS_STATUS_CODES_
/* capi.hpp:41-47 */
enum {
  VK_OK = 0,
  VK_ERROR_INVALID_ARGUMENT = 1,
  VK_ERROR_OUT_OF_RANGE = 2,
  VK_ERROR_UNSUPPORTED = 3,
  VK_ERROR_INTERNAL = 4
};
#endif

/* capi.hpp:52-71, capi.cpp:30-47: thread-local; the message is valid until the
 * next failing call on the thread. */
const char* vk_last_error(void);
int vk_last_error_code(void);
void vk_set_last_error(int code, const char* message);

/*
 * The fused layer on the CPU (capi.hpp:515-523, capi_moe.cpp:81-108;
 * kernels/moe_fused.cpp:566-603).  Rows are pre-sorted: sorted_ids [EM],
 * expert_ids [EM / 16] (the oracle's block is 16 rows), topk_w_sorted [EM] the
 * routing weight of every sorted row.  act_scratch [EM, ispp] bf16, out
 * [M, hidden] fp32 zeroed by the caller and accumulated into.  group_size is
 * the block-scale group along K (32).  b13 / b2 may be null.  activation:
 * 0 = SwiGLU, 1 = SiTU.  The buffers are checked for null only when M > 0 and
 * EM > 0 (VK_ERROR_INVALID_ARGUMENT); shapes are the caller's to validate.
 */
int32_t vk_fused_moe_mxfp4(const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
                           const uint8_t* w2, const uint8_t* w2_scale, const int32_t* sorted_ids,
                           const float* topk_w_sorted, const int32_t* expert_ids,
                           uint16_t* act_scratch, float* out, int M, int hidden, int ispp, int top_k,
                           int EM, int group_size, float swiglu_limit, int activation, float beta,
                           float linear_beta, const float* b13, const float* b2);

/*
 * Block alignment of the routing table (capi.hpp:530-534, capi_moe.cpp:119-140;
 * kernels/moe_fused.cpp:609-661).  sorted_ids must hold
 * vk_moe_align_block_size_max_em(...) entries and expert_ids that many /
 * block_size; on success *out_EM is the padded row count.  Refused with
 * VK_ERROR_INVALID_ARGUMENT: block_size <= 0, num_experts < 0, M or top_k < 0,
 * out_EM null, and null buffers when M > 0.
 */
int32_t vk_moe_align_block_size(const int32_t* topk_ids, int32_t M, int32_t top_k, int32_t block_size,
                                int32_t num_experts, int32_t* sorted_ids, int32_t* expert_ids,
                                int32_t* out_EM);

/* capi.hpp:536-539, capi_moe.cpp:110-117: ((M top_k + bs - 1) / bs + num_experts) bs in
 * int32 arithmetic, 0 for a block size that is not positive.  (The device library
 * exports the same function.) */
size_t vk_moe_align_block_size_max_em(int32_t M, int32_t top_k, int32_t block_size, int32_t num_experts);

/*
 * MXFP4 orchestration ops (capi.hpp:470-503, capi_moe.cpp:20-75;
 * kernels/moe_aux.cpp:146-321).  Each refuses null buffers, negative sizes,
 * top_k <= 0, group_size <= 0, an odd hidden / width, and a hidden / width that
 * is not a multiple of group_size with VK_ERROR_INVALID_ARGUMENT, as the
 * reference's checks do (moe_aux.cpp:148-155, 211-215, 236-240, 261-266, 288-298).
 */
int32_t vk_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int M, int hidden,
                           int group_size);
int32_t vk_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int M,
                          int hidden, int top_k, int EM);
int32_t vk_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids, uint8_t* scales_sorted,
                                 int M, int n_groups, int top_k, int EM);
int32_t vk_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w, const int32_t* sorted_ids,
                                    float* out, int M, int width, int top_k, int EM);
int32_t vk_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                      const float* topk_w, const int32_t* sorted_ids, float* out, int M,
                                      int width, int top_k, int EM, int group_size);

#ifdef __cplusplus
}
#endif

#endif /* VKERNELS_CPU_H_ */
