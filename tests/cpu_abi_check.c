/*
 * cpu_abi_check.c — a C consumer of the host-side ABI declared in
 * include/vkernels_cpu.h, linked against the CPU checker (oracle/liboracle.so).
 *
 * Restates, through that header alone, the known-answer cases the reference holds for
 * its CPU ABI (tests/capi/test_capi.cpp:1480-1630: align example and null guard, the
 * all-ones layer with its closed form, SiTU, null buffers) and for the orchestration
 * ops (tests/kernels/moe/test_moe_aux.cpp: quantiser table values, sort, scatter).
 * Exit status 0 = every check held; otherwise the failed lines are printed.
 * Built and run by tests/test_cpu_abi.py; no GPU involved.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "vkernels_cpu.h"

static int failures = 0;
#define CHECK(cond)                                                   \
  do {                                                                \
    if (!(cond)) {                                                    \
      printf("%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      ++failures;                                                     \
    }                                                                 \
  } while (0)

static uint16_t bf16(float x) {
  uint32_t b;
  memcpy(&b, &x, 4);
  return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}

static void align_example(void) {
  /* 8 tokens, top-4, 4 experts: 5, 11 and 16 rows -> three blocks of 16, EM = 48 */
  enum { M = 8, K = 4, E = 4, BS = 16, N = M * K };
  int32_t ids[N];
  for (int i = 0; i < N; ++i) ids[i] = i < 5 ? 0 : i < 16 ? 1 : 2;
  const size_t max_em = vk_moe_align_block_size_max_em(M, K, BS, E);
  CHECK(max_em == (size_t)((N + BS - 1) / BS + E) * BS);
  CHECK(vk_moe_align_block_size_max_em(M, K, 0, E) == 0);
  int32_t* sids = malloc(sizeof(int32_t) * max_em);
  int32_t* eids = malloc(sizeof(int32_t) * max_em / BS);
  int32_t em = -1;
  CHECK(vk_moe_align_block_size(ids, M, K, BS, E, sids, eids, &em) == VK_OK);
  CHECK(em == 48);
  CHECK(eids[0] == 0 && eids[1] == 1 && eids[2] == 2);
  for (int i = 0; i < 5; ++i) CHECK(sids[i] == i);
  for (int i = 5; i < 16; ++i) CHECK(sids[i] == N);       /* padding = M * top_k */
  for (int i = 0; i < 11; ++i) CHECK(sids[16 + i] == 5 + i);
  for (int i = 0; i < 16; ++i) CHECK(sids[32 + i] == 16 + i);
  /* guards */
  CHECK(vk_moe_align_block_size(NULL, 1, 1, 16, 4, NULL, NULL, &em) == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_last_error_code() == VK_ERROR_INVALID_ARGUMENT && vk_last_error()[0] != 0);
  CHECK(vk_moe_align_block_size(ids, M, K, 0, E, sids, eids, &em) == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_moe_align_block_size(ids, M, K, BS, -1, sids, eids, &em) == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_moe_align_block_size(ids, M, K, BS, E, sids, eids, NULL) == VK_ERROR_INVALID_ARGUMENT);
  free(sids);
  free(eids);
}

static void all_ones_layer(void) {
  /* A = 1, every weight 1.0 (code 2, scale byte 127): gate = up = 128, silu(128) = 128
   * in fp32, act = 16384, out = 64 * 16384 = 1048576, all exact */
  enum { M = 16, H = 128, I = 64, E = 1, BS = 16 };
  uint16_t A[M * H];
  for (int i = 0; i < M * H; ++i) A[i] = bf16(1.0f);
  uint8_t* w13 = malloc((size_t)E * 2 * I * H / 2);
  uint8_t* w13s = malloc((size_t)E * 2 * I * H / 32);
  uint8_t* w2 = malloc((size_t)E * H * I / 2);
  uint8_t* w2s = malloc((size_t)E * H * I / 32);
  memset(w13, 0x22, (size_t)E * 2 * I * H / 2);
  memset(w13s, 127, (size_t)E * 2 * I * H / 32);
  memset(w2, 0x22, (size_t)E * H * I / 2);
  memset(w2s, 127, (size_t)E * H * I / 32);
  int32_t ids[M];
  float tw[M];
  for (int i = 0; i < M; ++i) { ids[i] = 0; tw[i] = 1.0f; }
  const size_t max_em = vk_moe_align_block_size_max_em(M, 1, BS, E);
  int32_t* sids = malloc(sizeof(int32_t) * max_em);
  int32_t* eids = malloc(sizeof(int32_t) * max_em / BS);
  int32_t em = 0;
  CHECK(vk_moe_align_block_size(ids, M, 1, BS, E, sids, eids, &em) == VK_OK && em == 16);
  uint16_t act[M * I];
  float out[M * H];
  memset(act, 0, sizeof act);
  memset(out, 0, sizeof out);
  CHECK(vk_fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tw, eids, act, out, M, H, I, 1, em, 32, 0.0f, 0,
                           0.0f, 0.0f, NULL, NULL) == VK_OK);
  for (int i = 0; i < M * I; ++i) CHECK(act[i] == bf16(16384.0f));
  for (int i = 0; i < M * H; ++i) CHECK(out[i] == 1048576.0f);
  /* out accumulates: a second call doubles it */
  CHECK(vk_fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tw, eids, act, out, M, H, I, 1, em, 32, 0.0f, 0,
                           0.0f, 0.0f, NULL, NULL) == VK_OK);
  CHECK(out[0] == 2097152.0f);
  /* SiTU, beta 4, linear_beta 25 (the clamp is ignored): 4 tanh(32) sigmoid(128) 25 tanh(5.12) */
  memset(out, 0, sizeof out);
  CHECK(vk_fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tw, eids, act, out, M, H, I, 1, em, 32, 1.0f, 1,
                           4.0f, 25.0f, NULL, NULL) == VK_OK);
  const double expect = 4.0 * tanh(128.0 / 4.0) * (1.0 / (1.0 + exp(-128.0))) * 25.0 * tanh(128.0 / 25.0) * I;
  for (int i = 0; i < M * H; ++i) CHECK(fabs(out[i] - expect) < 1e-2 * expect);
  /* bias only: zero codes, b13 = 1 on gate and up, b2 = 3: act = silu(1), out = 3 */
  memset(w13, 0, (size_t)E * 2 * I * H / 2);
  memset(w2, 0, (size_t)E * H * I / 2);
  float b13[2 * I], b2[H];
  for (int i = 0; i < 2 * I; ++i) b13[i] = 1.0f;
  for (int i = 0; i < H; ++i) b2[i] = 3.0f;
  memset(out, 0, sizeof out);
  CHECK(vk_fused_moe_mxfp4(A, w13, w13s, w2, w2s, sids, tw, eids, act, out, M, H, I, 1, em, 32, 0.0f, 0,
                           0.0f, 0.0f, b13, b2) == VK_OK);
  for (int i = 0; i < M * H; ++i) CHECK(out[i] == 3.0f);
  CHECK(act[0] == bf16(1.0f / (1.0f + expf(-1.0f))));
  /* null buffers are refused when there is work, and only then */
  CHECK(vk_fused_moe_mxfp4(NULL, w13, w13s, w2, w2s, sids, tw, eids, act, out, M, H, I, 1, em, 32, 0.0f,
                           0, 0.0f, 0.0f, NULL, NULL) == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_last_error_code() == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_fused_moe_mxfp4(NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, 0, H, I, 1, 0, 32,
                           0.0f, 0, 0.0f, 0.0f, NULL, NULL) == VK_OK);
  free(w13); free(w13s); free(w2); free(w2s); free(sids); free(eids);
}

static void orchestration_ops(void) {
  /* one group of 32: amax = 3 -> scale 2^0 (byte 127); codes of the reference's table
   * {0, .25, 1, 1.5, 2, 3}, ties to the larger, sign bit 8 */
  enum { K = 32 };
  const float vals[8] = {3.0f, -1.5f, 0.25f, 0.0f, 1.25f, -0.125f, 2.5f, 0.6f};
  const uint8_t codes[8] = {5, 8 | 3, 1, 0, 3, 8 | 1, 5, 1};
  uint16_t A[2 * K];
  memset(A, 0, sizeof A);
  for (int i = 0; i < 8; ++i) A[i] = bf16(vals[i]);
  for (int i = 0; i < K; ++i) A[K + i] = bf16(96.0f);     /* amax 96 = 3 * 2^5: byte 132, code 5 */
  uint8_t packed[2 * K / 2], scales[2];
  CHECK(vk_mxfp4_moe_quant(A, packed, scales, 2, K, 32) == VK_OK);
  CHECK(scales[0] == 127 && scales[1] == 132);
  for (int i = 0; i < 8; ++i) CHECK(((packed[i / 2] >> (4 * (i & 1))) & 15) == codes[i]);
  for (int i = 0; i < K / 2; ++i) CHECK(packed[K / 2 + i] == 0x55);
  CHECK(vk_mxfp4_moe_quant(A, packed, scales, 2, K, 0) == VK_ERROR_INVALID_ARGUMENT);
  CHECK(vk_mxfp4_moe_quant(A, packed, scales, 2, 31, 31) == VK_ERROR_INVALID_ARGUMENT);   /* odd */
  CHECK(vk_mxfp4_moe_quant(NULL, packed, scales, 2, K, 32) == VK_ERROR_INVALID_ARGUMENT);
  /* sort: rows in sorted order, padding rows zero */
  const int32_t sids[4] = {1, 2, 0, 1};   /* M = 2, top_k = 1: ids 2 is padding (>= M top_k) */
  uint16_t sorted[4 * K];
  memset(sorted, 0xAB, sizeof sorted);
  CHECK(vk_mxfp4_moe_sort(A, sids, sorted, 2, K, 1, 4) == VK_OK);
  CHECK(memcmp(sorted, A + K, 2 * K) == 0 && memcmp(sorted + 2 * K, A, 2 * K) == 0);
  for (int i = 0; i < K; ++i) CHECK(sorted[K + i] == 0);
  uint8_t ssorted[4];
  CHECK(vk_mxfp4_moe_sort_scales(scales, sids, ssorted, 2, 1, 1, 4) == VK_OK);
  CHECK(ssorted[0] == 132 && ssorted[1] == 0 && ssorted[2] == 127 && ssorted[3] == 132);
  CHECK(vk_mxfp4_moe_sort(A, sids, sorted, 2, K, 0, 4) == VK_ERROR_INVALID_ARGUMENT);
  /* scatter: out[token] += partial[r] * w[r] over the routed rows in ascending order */
  float partial[4 * 2] = {1, 2, 100, 100, 3, 4, 5, 6};
  const float w[4] = {0.5f, 9.0f, 2.0f, 0.25f};
  float out[2 * 2] = {10, 10, 10, 10};
  CHECK(vk_mxfp4_moe_scatter_reduce(partial, w, sids, out, 2, 2, 1, 4) == VK_OK);
  CHECK(out[0] == 16.0f && out[1] == 18.0f && out[2] == 11.75f && out[3] == 12.5f);
  CHECK(vk_mxfp4_moe_scatter_reduce(partial, w, sids, NULL, 2, 2, 1, 4) == VK_ERROR_INVALID_ARGUMENT);
  /* the quantised form: codes 5 (= 3.0) with scale 2^5 -> 96 per value */
  uint8_t pq[4 * K / 2], ps[4];
  memset(pq, 0x55, sizeof pq);
  memset(ps, 132, sizeof ps);
  float outq[2 * K];
  memset(outq, 0, sizeof outq);
  CHECK(vk_mxfp4_moe_scatter_reduce_q(pq, ps, w, sids, outq, 2, K, 1, 4, 32) == VK_OK);
  CHECK(outq[0] == 192.0f && outq[K] == 72.0f && outq[2 * K - 1] == 72.0f);
  CHECK(vk_mxfp4_moe_scatter_reduce_q(pq, ps, w, sids, outq, 2, K, 1, 4, 24) == VK_ERROR_INVALID_ARGUMENT);
}

int main(void) {
  align_example();
  all_ones_layer();
  orchestration_ops();
  vk_set_last_error(VK_OK, "");
  CHECK(vk_last_error_code() == VK_OK && vk_last_error()[0] == 0);
  if (failures == 0) printf("cpu abi: all checks held\n");
  return failures == 0 ? 0 : 1;
}
