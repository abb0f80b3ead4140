/*
 * moe_oracle.c — CPU restatement of the reference's fused MXFP4 MoE oracle.
 * TEST INFRASTRUCTURE ONLY (see moe_oracle.h).
 *
 * The loops are organised differently from the reference (one weight-tile
 * dequantisation per run of same-expert blocks instead of one per 16-row
 * block, the inner product vectorised across output columns, OpenMP over
 * independent output tiles), but every output element is produced by the
 * same sequence of fp32 operations as in the reference:
 *
 *   for each 64-wide K block, in ascending order:
 *       dot = 0; for k in the block, ascending: dot += a[k] * w[k]
 *       acc += dot
 *
 * (src/c/vkernels/kernels/moe_fused.cpp:315-325).  Compile with
 * -ffp-contract=off so that no multiply-add is fused, as the reference's
 * build does (src/c/CMakeLists.txt:8-11).
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { BLK_M = 16, BLK_N = 64, BLK_K = 64 };

static int g_threads = 1;

void vko_set_threads(int n) { g_threads = n < 1 ? 1 : n; }

/* ---------------------------------------------------------------------- */
/* scalar decoders                                                         */
/* ---------------------------------------------------------------------- */

static inline float bits_to_float(uint32_t b) {
  float f;
  memcpy(&f, &b, sizeof f);
  return f;
}

static inline uint32_t float_to_bits(float f) {
  uint32_t b;
  memcpy(&b, &f, sizeof b);
  return b;
}

/* moe_fused.cpp:24-39 */
uint32_t vko_fp4nib_to_f32bits(int nibble) {
  const uint32_t sign = (nibble & 8) ? 0x80000000u : 0u;
  const int e = (nibble >> 1) & 3;
  const int m = nibble & 1;
  switch (e) {
    case 0:
      return m ? (sign | 0x3E800000u) : sign; /* +-0.25, +-0 */
    case 3:
      return m ? 0x7FC00000u : (sign | 0x7F800000u); /* NaN, +-inf */
    default:
      return sign | ((uint32_t)(126 + e) << 23) | (m ? 0x00400000u : 0u);
  }
}

/* moe_fused.cpp:50-64 */
float vko_ue8m0_to_float(uint8_t s) {
  if (s == 0xFF) return 0.0f;
  if (s == 0) return bits_to_float(0x00400000u); /* 2^-127 */
  return bits_to_float((uint32_t)s << 23);
}

/* moe_fused.cpp:41-45 */
uint16_t vko_f32bits_to_bf16(uint32_t bits) {
  bits += 0x7FFFu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

static inline float bf16_to_float(uint16_t v) {
  return bits_to_float((uint32_t)v << 16);
}

/* ---------------------------------------------------------------------- */
/* optional model of the GPU's activation operands (NOT in the reference)  */
/* ---------------------------------------------------------------------- */

/*
 * The prefill kernels feed the matrix cores the bf16 activations as a sum of
 * FP6 (E2M3) terms per block of 32 along K: with e the largest exponent field
 * of the block and s = 2^(e-2-127),
 *     t0 = Q(a / s) * s,  t1 = Q((a - t0) / (s/16)) * (s/16),
 *     t2 = Q((a - t0 - t1) / (s/256)) * (s/256),          a' = t0 + t1 (+ t2),
 * Q = round to nearest even on the E2M3 grid, saturating at +-7.5.  With the
 * model switched on (terms = 2 or 3) the grouped GEMMs multiply a' instead of
 * a, so a test can tell the error of that representation (model vs reference
 * arithmetic, both on the CPU) from the error of the GPU's accumulation (GPU
 * vs model).  terms = 1 is the W4A4 mode: the activations are quantised to
 * MXFP4 as the reference's mxfp4_moe_quant does (aux_oracle.c) and dequantised.
 * terms = 0, the default, is the reference's arithmetic.
 */
static int g_act_model = 0;

static int g_act_model_down = 0; /* the second stage's, when it differs (terms = first + 16 * second) */

void vko_set_act_model(int terms) {
  const int first = terms & 15, second = terms >> 4;
  g_act_model = (first >= 1 && first <= 3) ? first : 0;
  g_act_model_down = (second >= 1 && second <= 3) ? second : g_act_model;
}

static float e2m3_round(float v) {
  const float a = fabsf(v);
  float q;
  if (a < 2.0f) q = nearbyintf(a * 8.0f) * 0.125f;        /* subnormals and [1, 2): steps of 1/8 */
  else if (a < 4.0f) q = nearbyintf(a * 4.0f) * 0.25f;
  else q = nearbyintf(a * 2.0f) * 0.5f;
  if (q > 7.5f) q = 7.5f;
  return v < 0.0f ? -q : q;
}

/* a' for one block of 32 bf16 values (finite; blocks of zeros stay zeros).  Every term
 * has a scale of its own, set as the first one's is: from the largest exponent field of
 * what the terms before it left (exact in bf16), less 2, and not below 2^(64-127). */
void vko_act_model_block32(const uint16_t* a, float* out, int terms) {
  float rest[32];
  for (int k = 0; k < 32; ++k) {
    rest[k] = bits_to_float((uint32_t)a[k] << 16);
    out[k] = 0.0f;
  }
  for (int t = 0; t < terms; ++t) {
    int emax = 0;
    for (int k = 0; k < 32; ++k) {
      const int e = (int)((float_to_bits(rest[k]) >> 23) & 0xFF); /* bf16 and fp32 share the exponent field */
      if (e > emax) emax = e;
    }
    if (emax == 0) break; /* nothing left (bf16 subnormals count as zero) */
    int sb = emax - 2;
    if (sb < 64) sb = 64;
    const float st = ldexpf(1.0f, sb - 127);
    for (int k = 0; k < 32; ++k) {
      const float term = e2m3_round(rest[k] / st) * st; /* exact: a few bits of the value */
      out[k] += term;
      rest[k] -= term;
    }
  }
}

/* ---------------------------------------------------------------------- */
/* weight-tile dequantisation                                              */
/* ---------------------------------------------------------------------- */

/* moe_fused.cpp:183-201: one scale decode and two nibble decodes per byte. */
void vko_dequant_weight_tile_ref(const uint8_t* packed, const uint8_t* scale,
                                 uint16_t* out_bf16, int N, int K,
                                 int group_size, int stride_packed,
                                 int stride_scale_n, int stride_scale_k) {
  for (int n = 0; n < N; ++n) {
    for (int kp = 0; kp < K / 2; ++kp) {
      const uint8_t pb = packed[(size_t)n * stride_packed + kp];
      const int g = (2 * kp) / group_size;
      const float sc = vko_ue8m0_to_float(
          scale[(size_t)n * stride_scale_n + (size_t)g * stride_scale_k]);
      const float lo = bits_to_float(vko_fp4nib_to_f32bits(pb & 15)) * sc;
      const float hi = bits_to_float(vko_fp4nib_to_f32bits(pb >> 4)) * sc;
      out_bf16[(size_t)(2 * kp) * N + n] = vko_f32bits_to_bf16(float_to_bits(lo));
      out_bf16[(size_t)(2 * kp + 1) * N + n] =
          vko_f32bits_to_bf16(float_to_bits(hi));
    }
  }
}

/* moe_fused.cpp:141-174: the same values through two lookup tables. */
void vko_dequant_weight_tile(const uint8_t* packed, const uint8_t* scale,
                             uint16_t* out_bf16, int N, int K, int group_size,
                             int stride_packed, int stride_scale_n,
                             int stride_scale_k) {
  float nib[16];
  for (int i = 0; i < 16; ++i) nib[i] = bits_to_float(vko_fp4nib_to_f32bits(i));
  for (int n = 0; n < N; ++n) {
    const uint8_t* prow = packed + (size_t)n * stride_packed;
    const uint8_t* srow = scale + (size_t)n * stride_scale_n;
    for (int k0 = 0; k0 < K; k0 += group_size) {
      const float sc =
          vko_ue8m0_to_float(srow[(size_t)(k0 / group_size) * stride_scale_k]);
      const int k1 = (k0 + group_size < K) ? k0 + group_size : K;
      for (int k = k0; k < k1; k += 2) {
        const uint8_t pb = prow[k / 2];
        out_bf16[(size_t)k * N + n] =
            vko_f32bits_to_bf16(float_to_bits(nib[pb & 15] * sc));
        out_bf16[(size_t)(k + 1) * N + n] =
            vko_f32bits_to_bf16(float_to_bits(nib[pb >> 4] * sc));
      }
    }
  }
}

/* ---------------------------------------------------------------------- */
/* grouped GEMM shared by stage 0a and stage 1a                            */
/* ---------------------------------------------------------------------- */

typedef struct {
  int first_block; /* index of the first 16-row block of the run */
  int num_blocks;  /* consecutive blocks with the same expert id  */
  int expert;
} run_t;

static int collect_runs(const int32_t* expert_ids, int num_blocks, run_t* runs) {
  int n = 0;
  int b = 0;
  while (b < num_blocks) {
    const int e = expert_ids[b];
    if (e < 0) {
      ++b;
      continue;
    }
    int len = 1;
    while (b + len < num_blocks && expert_ids[b + len] == e) ++len;
    runs[n].first_block = b;
    runs[n].num_blocks = len;
    runs[n].expert = e;
    ++n;
    b += len;
  }
  return n;
}

/*
 * C[r, 0:n_out] = Arow(r)[k_base : k_base+k_dim] . W[e, 0:n_out, 0:k_dim]^T
 * for every sorted row r of every block with expert_ids >= 0; padding rows
 * of such blocks get zeros, blocks with expert_ids < 0 are not touched.
 *
 * gather != 0: Arow(r) = A[(sorted_ids[r] / top_k) * a_stride]   (stage 0a)
 * gather == 0: Arow(r) = A[r * a_stride]                         (stage 1a)
 */
static void grouped_gemm(const uint16_t* A, int gather, const uint8_t* W,
                         const uint8_t* Ws, const int32_t* sorted_ids,
                         const int32_t* expert_ids, float* C, int n_flat,
                         int top_k, int EM, int a_stride, int k_base, int k_dim,
                         int n_out, int group_size) {
  const int num_blocks = EM / BLK_M;
  if (num_blocks <= 0 || n_out <= 0) return;
  const int n_tiles = n_out / BLK_N;
  const int k_tiles = k_dim / BLK_K;
  const size_t w_expert_bytes = (size_t)n_out * (size_t)(k_dim / 2);
  const size_t ws_expert_bytes = (size_t)n_out * (size_t)(k_dim / group_size);

  run_t* runs = (run_t*)malloc(sizeof(run_t) * (size_t)num_blocks);
  const int n_runs = collect_runs(expert_ids, num_blocks, runs);
  const long n_jobs = (long)n_runs * n_tiles;

#pragma omp parallel num_threads(g_threads)
  {
    uint16_t* tile_bf = (uint16_t*)malloc(sizeof(uint16_t) * BLK_K * BLK_N);
    float* tile_f = (float*)malloc(sizeof(float) * BLK_K * BLK_N);
    float* acc = NULL;
    size_t acc_rows = 0;

#pragma omp for schedule(dynamic, 1)
    for (long job = 0; job < n_jobs; ++job) {
      const run_t run = runs[job / n_tiles];
      const int nt = (int)(job % n_tiles);
      const int row0 = run.first_block * BLK_M;
      const int rows = run.num_blocks * BLK_M;
      if ((size_t)rows > acc_rows) {
        free(acc);
        acc = (float*)malloc(sizeof(float) * (size_t)rows * BLK_N);
        acc_rows = (size_t)rows;
      }
      memset(acc, 0, sizeof(float) * (size_t)rows * BLK_N);

      const uint8_t* w_tile = W + (size_t)run.expert * w_expert_bytes +
                              (size_t)nt * BLK_N * (size_t)(k_dim / 2);
      const uint8_t* s_tile = Ws + (size_t)run.expert * ws_expert_bytes +
                              (size_t)nt * BLK_N * (size_t)(k_dim / group_size);

      for (int kt = 0; kt < k_tiles; ++kt) {
        const int k0 = kt * BLK_K;
        vko_dequant_weight_tile(w_tile + k0 / 2, s_tile + k0 / group_size,
                                tile_bf, BLK_N, BLK_K, group_size, k_dim / 2,
                                k_dim / group_size, 1);
        for (int i = 0; i < BLK_K * BLK_N; ++i) tile_f[i] = bf16_to_float(tile_bf[i]);

        for (int r = 0; r < rows; ++r) {
          const int flat = sorted_ids[row0 + r];
          if (flat >= n_flat) continue; /* padding row contributes nothing */
          const uint16_t* arow =
              gather ? A + (size_t)(flat / top_k) * a_stride + k_base + k0
                     : A + (size_t)(row0 + r) * a_stride + k_base + k0;
          float dot[BLK_N];
          float amodel[BLK_K];
          const int model = gather ? g_act_model : g_act_model_down;
          if (model == 1) {
            vko_aux_model_block32(arow, amodel);
            vko_aux_model_block32(arow + 32, amodel + 32);
          } else if (model != 0) {
            vko_act_model_block32(arow, amodel, model);
            vko_act_model_block32(arow + 32, amodel + 32, model);
          }
          for (int n = 0; n < BLK_N; ++n) dot[n] = 0.0f;
          for (int k = 0; k < BLK_K; ++k) {
            const float a = model != 0 ? amodel[k] : bf16_to_float(arow[k]);
            const float* wrow = tile_f + (size_t)k * BLK_N;
            for (int n = 0; n < BLK_N; ++n) dot[n] += a * wrow[n];
          }
          float* arow_acc = acc + (size_t)r * BLK_N;
          for (int n = 0; n < BLK_N; ++n) arow_acc[n] += dot[n];
        }
      }

      for (int r = 0; r < rows; ++r)
        memcpy(C + (size_t)(row0 + r) * n_out + (size_t)nt * BLK_N,
               acc + (size_t)r * BLK_N, sizeof(float) * BLK_N);
    }
    free(acc);
    free(tile_f);
    free(tile_bf);
  }
  free(runs);
}

/* moe_fused.cpp:235-365.  gate columns are w13 rows [0,ispp), up columns are
 * w13 rows [ispp,2*ispp): output column == weight row. */
void vko_moe_gateup(const uint16_t* A, const uint8_t* w13,
                    const uint8_t* w13_scale, const int32_t* sorted_ids,
                    const int32_t* expert_ids, float* gate_up, int M,
                    int a_stride, int k_base, int hidden_k, int ispp,
                    int top_k, int EM, int group_size) {
  grouped_gemm(A, 1, w13, w13_scale, sorted_ids, expert_ids, gate_up,
               M * top_k, top_k, EM, a_stride, k_base, hidden_k, 2 * ispp,
               group_size);
}

/* moe_fused.cpp:427-518 */
void vko_moe_down(const uint16_t* act, const uint8_t* w2,
                  const uint8_t* w2_scale, const int32_t* sorted_ids,
                  const int32_t* expert_ids, float* partial, int M,
                  int a_stride, int k_base, int ispp_k, int hidden, int top_k,
                  int EM, int group_size) {
  grouped_gemm(act, 0, w2, w2_scale, sorted_ids, expert_ids, partial,
               M * top_k, top_k, EM, a_stride, k_base, ispp_k, hidden,
               group_size);
}

/* ---------------------------------------------------------------------- */
/* epilogues                                                               */
/* ---------------------------------------------------------------------- */

/* moe_fused.cpp:206-226 */
float vko_epilogue_value(int activation, float g, float u, float swiglu_limit,
                         float beta, float linear_beta) {
  if (activation == VKO_SITU) {
    const float sig = 1.0f / (1.0f + expf(-g));
    const float gate_out = beta * tanhf(g / beta) * sig;
    const float up_out =
        (linear_beta > 0.0f) ? linear_beta * tanhf(u / linear_beta) : u;
    return gate_out * up_out;
  }
  if (swiglu_limit > 0.0f) {
    if (g > swiglu_limit) g = swiglu_limit;
    if (u > swiglu_limit) u = swiglu_limit;
    if (u < -swiglu_limit) u = -swiglu_limit;
  }
  const float silu = g / (1.0f + expf(-g));
  return silu * u;
}

/* moe_fused.cpp:370-422 */
void vko_moe_act_epilogue(const float* gate_up, const float* b13,
                          uint16_t* act, const int32_t* sorted_ids,
                          const int32_t* expert_ids, int M, int top_k, int EM,
                          int ispp, float swiglu_limit, int activation,
                          float beta, float linear_beta) {
  const int n_flat = M * top_k;
  const int num_blocks = EM / BLK_M;
  const int cols = (ispp / BLK_N) * BLK_N;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int b = 0; b < num_blocks; ++b) {
    const int e = expert_ids[b];
    if (e < 0) continue;
    for (int m = 0; m < BLK_M; ++m) {
      const size_t r = (size_t)b * BLK_M + m;
      if (sorted_ids[r] >= n_flat) continue;
      const float* gu = gate_up + r * (size_t)(2 * ispp);
      const float* bias = b13 ? b13 + (size_t)e * (size_t)(2 * ispp) : NULL;
      for (int n = 0; n < cols; ++n) {
        float g = gu[n];
        float u = gu[ispp + n];
        if (bias) {
          g += bias[n];
          u += bias[ispp + n];
        }
        const float v = vko_epilogue_value(activation, g, u, swiglu_limit,
                                           beta, linear_beta);
        act[r * (size_t)ispp + n] = vko_f32bits_to_bf16(float_to_bits(v));
      }
    }
  }
}

/* moe_fused.cpp:523-564.  Rows are visited in ascending sorted order, so the
 * contributions of one token are added in ascending block order. */
void vko_moe_combine(const float* partial, const float* b2,
                     const float* topk_w_sorted, const int32_t* sorted_ids,
                     const int32_t* expert_ids, float* out, int M, int hidden,
                     int top_k, int EM) {
  const int n_flat = M * top_k;
  const int num_blocks = EM / BLK_M;
  const int cols = (hidden / BLK_N) * BLK_N;
  for (int b = 0; b < num_blocks; ++b) {
    const int e = expert_ids[b];
    if (e < 0) continue;
    for (int m = 0; m < BLK_M; ++m) {
      const size_t r = (size_t)b * BLK_M + m;
      const int flat = sorted_ids[r];
      if (flat >= n_flat) continue;
      const float w = topk_w_sorted[r];
      const float* p = partial + r * (size_t)hidden;
      const float* bias = b2 ? b2 + (size_t)e * (size_t)hidden : NULL;
      float* o = out + (size_t)(flat / top_k) * (size_t)hidden;
      for (int n = 0; n < cols; ++n) {
        float v = p[n];
        if (bias) v += bias[n];
        v *= w;
        o[n] += v;
      }
    }
  }
}

/* moe_fused.cpp:569-603 */
void vko_fused_moe_mxfp4(const uint16_t* A, const uint8_t* w13,
                         const uint8_t* w13_scale, const uint8_t* w2,
                         const uint8_t* w2_scale, const int32_t* sorted_ids,
                         const float* topk_w_sorted, const int32_t* expert_ids,
                         uint16_t* act_scratch, float* out, int M, int hidden,
                         int ispp, int top_k, int EM, int group_size,
                         float swiglu_limit, int activation, float beta,
                         float linear_beta, const float* b13, const float* b2) {
  if (EM <= 0) return;
  float* gate_up = (float*)malloc(sizeof(float) * (size_t)EM * 2 * (size_t)ispp);
  float* partial = (float*)malloc(sizeof(float) * (size_t)EM * (size_t)hidden);
  vko_moe_gateup(A, w13, w13_scale, sorted_ids, expert_ids, gate_up, M, hidden,
                 0, hidden, ispp, top_k, EM, group_size);
  vko_moe_act_epilogue(gate_up, b13, act_scratch, sorted_ids, expert_ids, M,
                       top_k, EM, ispp, swiglu_limit, activation, beta,
                       linear_beta);
  vko_moe_down(act_scratch, w2, w2_scale, sorted_ids, expert_ids, partial, M,
               ispp, 0, ispp, hidden, top_k, EM, group_size);
  vko_moe_combine(partial, b2, topk_w_sorted, sorted_ids, expert_ids, out, M,
                  hidden, top_k, EM);
  free(partial);
  free(gate_up);
}

/* ---------------------------------------------------------------------- */
/* alignment                                                               */
/* ---------------------------------------------------------------------- */

static int round_up(int v, int m) { return (v + m - 1) / m * m; }

/* Stable counting sort of the flat indices by (local) expert.  `local_of`
 * returns the bucket of flat index i or -1 to drop it. */
static int align_core(const int32_t* topk_ids, const int32_t* expert_map,
                      int n_flat, int block_size, int num_experts, int buckets,
                      int32_t* sorted_ids, int32_t* expert_ids, int limit) {
  int* count = (int*)calloc((size_t)buckets + 1, sizeof(int));
  int* start = (int*)calloc((size_t)buckets + 1, sizeof(int));
  for (int i = 0; i < n_flat; ++i) {
    const int ge = topk_ids[i];
    if (ge < 0 || ge >= num_experts) continue;
    const int le = expert_map ? expert_map[ge] : ge;
    if (le < 0 || le >= buckets) continue;
    ++count[le];
  }
  int em = 0;
  for (int e = 0; e < buckets; ++e) {
    start[e] = em;
    em += round_up(count[e], block_size);
  }
  /* padding sentinel for the rows of every expert's last partial block, and
   * the expert id of every block that holds at least one real row */
  int blk = 0;
  for (int e = 0; e < buckets; ++e) {
    const int padded = round_up(count[e], block_size);
    for (int i = count[e]; i < padded; ++i)
      if (start[e] + i < limit) sorted_ids[start[e] + i] = n_flat;
    for (int b = 0; b < padded / block_size; ++b, ++blk)
      if (blk < limit / block_size)
        expert_ids[blk] = (b * block_size < count[e]) ? e : -1;
  }
  for (int i = 0; i < n_flat; ++i) {
    const int ge = topk_ids[i];
    if (ge < 0 || ge >= num_experts) continue;
    const int le = expert_map ? expert_map[ge] : ge;
    if (le < 0 || le >= buckets) continue;
    const int pos = start[le]++;
    if (pos < limit) sorted_ids[pos] = i;
  }
  free(start);
  free(count);
  return em;
}

/* moe_fused.cpp:609-661: only the first EM / EM/block_size entries are
 * written; EM is 0 when nothing routes. */
int vko_moe_align_block_size(const int32_t* topk_ids, int M, int top_k,
                             int block_size, int num_experts,
                             int32_t* sorted_ids, int32_t* expert_ids) {
  return align_core(topk_ids, NULL, M * top_k, block_size, num_experts,
                    num_experts, sorted_ids, expert_ids, 0x7FFFFFFF);
}

/* vllm_experts.py:297-372 / moe_fused.hip:1983-2071 */
int vko_moe_align_block_size_with_map(const int32_t* topk_ids,
                                      const int32_t* expert_map, int N,
                                      int block_size, int num_experts,
                                      int local_n, int max_EM,
                                      int32_t* sorted_ids,
                                      int32_t* expert_ids) {
  for (int i = 0; i < max_EM; ++i) sorted_ids[i] = N;
  for (int i = 0; i < max_EM / block_size; ++i) expert_ids[i] = -1;
  int em = align_core(topk_ids, expert_map, N, block_size, num_experts,
                      local_n, sorted_ids, expert_ids, max_EM);
  if (em == 0) em = block_size;
  if (em > max_EM) em = max_EM;
  return em;
}

/* capi/capi_moe.cpp:110-117 */
size_t vko_align_max_em(int M, int top_k, int block_size, int num_experts) {
  if (block_size <= 0) return 0;
  const int32_t n = M * top_k;
  const int32_t v = ((n + block_size - 1) / block_size + num_experts) * block_size;
  return v > 0 ? (size_t)v : 0;
}

/* vllm_experts.py:481-500 */
int vko_align_em_bound(int M, int top_k, int local_n, int block_size) {
  const int n = M * top_k;
  if (n <= 0) return block_size;
  const int head = (n < local_n ? n : local_n) * block_size;
  if (n <= local_n) return head;
  return head + round_up(n - local_n, block_size);
}
