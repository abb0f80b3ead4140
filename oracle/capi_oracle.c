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
 *   vk_last_error / vk_last_error_code / vk_set_last_error
 *                                     src/c/vkernels/capi/capi.cpp:30-47
 */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "moe_oracle.h"

enum {
  VK_OK = 0,
  VK_ERROR_INVALID_ARGUMENT = 1,
  VK_ERROR_OUT_OF_RANGE = 2,
  VK_ERROR_UNSUPPORTED = 3,
  VK_ERROR_INTERNAL = 4
};

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
