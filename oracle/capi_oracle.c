/*
 * capi_oracle.c — the reference's CPU C ABI for the MoE path, served by the
 * oracle.  TEST INFRASTRUCTURE ONLY (see moe_oracle.h).
 *
 * Same names, argument order, status codes and null-guard behaviour as the
 * reference's host library, so that a test written against the reference's
 * CPU ABI runs unchanged against liboracle:
 *   vk_fused_moe_mxfp4                src/c/vkernels/capi/capi_moe.cpp:81-108
 *   vk_moe_align_block_size           src/c/vkernels/capi/capi_moe.cpp:119-140
 *   vk_moe_align_block_size_max_em    src/c/vkernels/capi/capi_moe.cpp:110-117
 *   vk_mxfp4_moe_quant / _sort / _sort_scales / _scatter_reduce / _scatter_reduce_q
 *                                     src/c/vkernels/capi/capi_moe.cpp:20-75, with the
 *                                     argument checks of kernels/moe_aux.cpp:148-298
 *   vk_last_error / vk_last_error_code / vk_set_last_error
 *                                     src/c/vkernels/capi/capi.cpp:30-47
 * The prototypes come from include/vkernels_cpu.h, so the compiler holds the
 * definitions below to the declared ABI.
 */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "moe_oracle.h"
#include "vkernels_cpu.h"

static _Thread_local char g_msg[256];
static _Thread_local int g_code = VK_OK;

void vk_set_last_error(int code, const char* message) {
  g_code = code;
  snprintf(g_msg, sizeof g_msg, "%s", message ? message : "");
}
const char* vk_last_error(void) { return g_msg; }
int vk_last_error_code(void) { return g_code; }

static int32_t fail(int code, const char* message) {
  vk_set_last_error(code, message);
  return code;
}

int32_t vk_fused_moe_mxfp4(const uint16_t* A, const uint8_t* w13,
                           const uint8_t* w13_scale, const uint8_t* w2,
                           const uint8_t* w2_scale, const int32_t* sorted_ids,
                           const float* topk_w_sorted,
                           const int32_t* expert_ids, uint16_t* act_scratch,
                           float* out, int M, int hidden, int ispp, int top_k,
                           int EM, int group_size, float swiglu_limit,
                           int activation, float beta, float linear_beta,
                           const float* b13, const float* b2) {
  if (M > 0 && EM > 0) {
    if (!A || !w13 || !w13_scale || !w2 || !w2_scale || !sorted_ids ||
        !topk_w_sorted || !expert_ids || !act_scratch || !out)
      return fail(VK_ERROR_INVALID_ARGUMENT,
                  "fused_moe_mxfp4: buffers must not be null");
  }
  vko_fused_moe_mxfp4(A, w13, w13_scale, w2, w2_scale, sorted_ids,
                      topk_w_sorted, expert_ids, act_scratch, out, M, hidden,
                      ispp, top_k, EM, group_size, swiglu_limit, activation,
                      beta, linear_beta, b13, b2);
  return VK_OK;
}

size_t vk_moe_align_block_size_max_em(int32_t M, int32_t top_k,
                                      int32_t block_size,
                                      int32_t num_experts) {
  return vko_align_max_em(M, top_k, block_size, num_experts);
}

int32_t vk_moe_align_block_size(const int32_t* topk_ids, int32_t M,
                                int32_t top_k, int32_t block_size,
                                int32_t num_experts, int32_t* sorted_ids,
                                int32_t* expert_ids, int32_t* out_EM) {
  if (block_size <= 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "block_size must be positive");
  if (num_experts < 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "num_experts must be non-negative");
  if (M < 0 || top_k < 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "M and top_k must be non-negative");
  if (!out_EM) return fail(VK_ERROR_INVALID_ARGUMENT, "out_EM must not be null");
  if (M > 0 && (!topk_ids || !sorted_ids || !expert_ids))
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "topk_ids/sorted_ids/expert_ids must not be null");
  *out_EM = vko_moe_align_block_size(topk_ids, M, top_k, block_size,
                                     num_experts, sorted_ids, expert_ids);
  return VK_OK;
}

/* ---- MXFP4 orchestration ops: the checks of the reference's functions
 * (VK_EXPECTS -> std::invalid_argument -> VK_ERROR_INVALID_ARGUMENT), then the oracle's
 * restatement of their bodies (aux_oracle.c). ---- */
#define EXPECT(cond, msg) \
  do { if (!(cond)) return fail(VK_ERROR_INVALID_ARGUMENT, msg); } while (0)

/* capi_moe.cpp:20-28, moe_aux.cpp:146-166 */
int32_t vk_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int M, int hidden,
                           int group_size) {
  EXPECT(A != NULL, "A must not be null");
  EXPECT(packed != NULL, "packed must not be null");
  EXPECT(scales != NULL, "scales must not be null");
  EXPECT(M >= 0 && hidden >= 0, "M and hidden must be non-negative");
  EXPECT(group_size > 0, "group_size must be positive");
  EXPECT(hidden % group_size == 0, "hidden must be a multiple of group_size");
  EXPECT(hidden % 2 == 0, "hidden must be even (two nibbles per byte)");
  vko_mxfp4_moe_quant(A, packed, scales, M, hidden, group_size);
  return VK_OK;
}

/* capi_moe.cpp:30-39, moe_aux.cpp:209-234 */
int32_t vk_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int M,
                          int hidden, int top_k, int EM) {
  EXPECT(A != NULL, "A must not be null");
  EXPECT(sorted_ids != NULL, "sorted_ids must not be null");
  EXPECT(A_sorted != NULL, "A_sorted must not be null");
  EXPECT(M >= 0 && hidden >= 0 && top_k > 0 && EM >= 0, "M, hidden, top_k, EM must be valid");
  vko_mxfp4_moe_sort(A, sorted_ids, A_sorted, M, hidden, top_k, EM);
  return VK_OK;
}

/* capi_moe.cpp:41-51, moe_aux.cpp:236-260 */
int32_t vk_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids, uint8_t* scales_sorted,
                                 int M, int n_groups, int top_k, int EM) {
  EXPECT(scales != NULL, "scales must not be null");
  EXPECT(sorted_ids != NULL, "sorted_ids must not be null");
  EXPECT(scales_sorted != NULL, "scales_sorted must not be null");
  EXPECT(M >= 0 && n_groups >= 0 && top_k > 0 && EM >= 0, "M, n_groups, top_k, EM must be valid");
  vko_mxfp4_moe_sort_scales(scales, sorted_ids, scales_sorted, M, n_groups, top_k, EM);
  return VK_OK;
}

/* capi_moe.cpp:53-62, moe_aux.cpp:261-285 */
int32_t vk_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w, const int32_t* sorted_ids,
                                    float* out, int M, int width, int top_k, int EM) {
  EXPECT(partial != NULL, "partial must not be null");
  EXPECT(topk_w != NULL, "topk_w must not be null");
  EXPECT(sorted_ids != NULL, "sorted_ids must not be null");
  EXPECT(out != NULL, "out must not be null");
  EXPECT(M >= 0 && width >= 0 && top_k > 0 && EM >= 0, "M, width, top_k, EM must be valid");
  vko_mxfp4_moe_scatter_reduce(partial, topk_w, sorted_ids, out, M, width, top_k, EM);
  return VK_OK;
}

/* capi_moe.cpp:64-75, moe_aux.cpp:288-321 */
int32_t vk_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                      const float* topk_w, const int32_t* sorted_ids, float* out, int M,
                                      int width, int top_k, int EM, int group_size) {
  EXPECT(partial_q != NULL, "partial_q must not be null");
  EXPECT(partial_s != NULL, "partial_s must not be null");
  EXPECT(topk_w != NULL, "topk_w must not be null");
  EXPECT(sorted_ids != NULL, "sorted_ids must not be null");
  EXPECT(out != NULL, "out must not be null");
  EXPECT(M >= 0 && width >= 0 && top_k > 0 && EM >= 0, "M, width, top_k, EM must be valid");
  EXPECT(group_size > 0, "group_size must be positive");
  EXPECT(width % 2 == 0, "width must be even (two nibbles per byte)");
  EXPECT(width % group_size == 0, "width must be a multiple of group_size");
  vko_mxfp4_moe_scatter_reduce_q(partial_q, partial_s, topk_w, sorted_ids, out, M, width, top_k, EM,
                                 group_size);
  return VK_OK;
}
