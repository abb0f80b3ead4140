/*
 * aux_oracle.c — CPU restatement of the reference's MXFP4 MoE orchestration
 * ops (activation quantisation, gathers, routed combine).
 * TEST INFRASTRUCTURE ONLY (see moe_oracle.h).
 *
 * Follows src/c/vkernels/kernels/moe_aux.cpp function by function; the
 * quantiser works on the bf16 bit patterns with integers where the reference
 * goes through float division and log2 (same results for every input: see
 * the comments; checked exhaustively against the compiled reference in
 * tests/test_oracle_aux.py).
 */
#include "moe_oracle.h"

#include <math.h>
#include <string.h>

static inline float bits_to_float(uint32_t b) {
  float f;
  memcpy(&f, &b, sizeof f);
  return f;
}

/* moe_aux.cpp:32-50 (the table of moe_fused.cpp:24-39) */
static float fp4_nibble_to_float(uint8_t nibble) {
  return bits_to_float(vko_fp4nib_to_f32bits(nibble & 15));
}

/* moe_aux.cpp:76-82: 0xFF -> 0, else bits s << 23 (so 0 -> +0.0, unlike the
 * weight decode of moe_fused.cpp, which maps 0 to 2^-127) */
static float aux_ue8m0_to_float(uint8_t s) {
  if (s == 0xFF) return 0.0f;
  return bits_to_float((uint32_t)s << 23);
}

/* moe_aux.cpp:62-73: nearest E2M1 magnitude, ties to the larger one; the sign
 * bit is set for x < 0 (so -0.0 keeps code 0 and a negative value that rounds
 * to zero becomes code 8). */
static uint8_t float_to_fp4_nib(float x) {
  const float v = fabsf(x);
  uint8_t mag;
  if (v < 0.125f) mag = 0;
  else if (v < 0.625f) mag = 1;
  else if (v < 1.25f) mag = 2;
  else if (v < 1.75f) mag = 3;
  else if (v < 2.5f) mag = 4;
  else mag = 5;
  if (x < 0.0f) mag |= 0x8;
  return mag;
}

/*
 * Scale byte of a group whose largest magnitude has the bf16 bit pattern
 * `amax_bits` (sign cleared).  moe_aux.cpp:108-131: zero or non-finite amax ->
 * 0xFF; else e = ceil(log2(amax / 3)), s = clamp(e + 127, 1, 254).
 * With amax = 1.m x 2^(x): amax / 3 lies in [2^(x-2) 1.33.., 2^(x-1) 1.33..), it
 * is a power of two only for m = 1.5, and the nearest other values are 2^-8
 * away in relative terms, so ceil(log2(.)) = x - 1 for m <= 1.5 and x above:
 * s = exponent field - (mantissa field <= 0x40).  bf16 subnormals give a
 * negative s, clamped to 1.
 */
uint8_t vko_aux_scale_byte(uint16_t amax_bits) {
  const int ex = (amax_bits >> 7) & 0xFF, mant = amax_bits & 0x7F;
  if (ex == 0xFF) return 0xFF;              /* inf or NaN */
  if (ex == 0 && mant == 0) return 0xFF;    /* zero */
  int s = ex - (mant <= 0x40 ? 1 : 0);
  if (ex == 0) s = 0;                       /* subnormal: e + 127 < 1 */
  if (s < 1) s = 1;
  if (s > 254) s = 254;
  return (uint8_t)s;
}

/* moe_aux.cpp:99-139 */
static void quant_row(const uint16_t* row, uint8_t* pk, uint8_t* sc, int hidden, int group_size) {
  const int n_groups = hidden / group_size;
  for (int g = 0; g < n_groups; ++g) {
    const int base = g * group_size;
    /* largest magnitude: the reference compares floats with `aa > amax` from 0, so a
     * NaN never becomes amax (the comparison is false) and an inf does */
    float amax = 0.0f;
    uint16_t amax_bits = 0;
    for (int i = 0; i < group_size; ++i) {
      const uint16_t b = (uint16_t)(row[base + i] & 0x7FFF);
      const float aa = bits_to_float((uint32_t)b << 16);
      if (aa > amax) {
        amax = aa;
        amax_bits = b;
      }
    }
    const uint8_t sb = vko_aux_scale_byte(amax_bits);
    sc[g] = sb;
    if (sb == 0xFF) {
      for (int kp = 0; kp < group_size / 2; ++kp) pk[base / 2 + kp] = 0;
      continue;
    }
    const float scale = aux_ue8m0_to_float(sb);
    for (int i = 0; i < group_size; i += 2) {
      const uint8_t lo = float_to_fp4_nib(bits_to_float((uint32_t)row[base + i] << 16) / scale);
      const uint8_t hi = float_to_fp4_nib(bits_to_float((uint32_t)row[base + i + 1] << 16) / scale);
      pk[base / 2 + i / 2] = (uint8_t)((hi << 4) | (lo & 0x0F));
    }
  }
}

/* moe_aux.cpp:146-166 */
void vko_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int M, int hidden,
                         int group_size) {
  for (int m = 0; m < M; ++m)
    quant_row(A + (size_t)m * hidden, packed + (size_t)m * (hidden / 2),
              scales + (size_t)m * (hidden / group_size), hidden, group_size);
}

/* moe_aux.cpp:171-209 */
void vko_mxfp4_moe_sorted_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed,
                                uint8_t* scales, int M, int hidden, int group_size, int top_k,
                                int EM) {
  const int n_groups = hidden / group_size;
  const int N = M * top_k;
  for (int r = 0; r < EM; ++r) {
    uint8_t* pk = packed + (size_t)r * (hidden / 2);
    uint8_t* sc = scales + (size_t)r * n_groups;
    const int flat = sorted_ids[r];
    if (flat >= 0 && flat < N) {
      quant_row(A + (size_t)(flat / top_k) * hidden, pk, sc, hidden, group_size);
    } else {
      memset(pk, 0, (size_t)hidden / 2);
      memset(sc, 0xFF, (size_t)n_groups);
    }
  }
}

/* moe_aux.cpp:214-234 */
void vko_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int M,
                        int hidden, int top_k, int EM) {
  const int N = M * top_k;
  for (int r = 0; r < EM; ++r) {
    uint16_t* dst = A_sorted + (size_t)r * hidden;
    const int flat = sorted_ids[r];
    if (flat >= 0 && flat < N) memcpy(dst, A + (size_t)(flat / top_k) * hidden, sizeof(uint16_t) * (size_t)hidden);
    else memset(dst, 0, sizeof(uint16_t) * (size_t)hidden);
  }
}

/* moe_aux.cpp:239-260 */
void vko_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids,
                               uint8_t* scales_sorted, int M, int n_groups, int top_k, int EM) {
  const int N = M * top_k;
  for (int r = 0; r < EM; ++r) {
    uint8_t* dst = scales_sorted + (size_t)r * n_groups;
    const int flat = sorted_ids[r];
    if (flat >= 0 && flat < N) memcpy(dst, scales + (size_t)(flat / top_k) * n_groups, (size_t)n_groups);
    else memset(dst, 0, (size_t)n_groups);
  }
}

/* moe_aux.cpp:265-285: ascending sorted row, out += partial * w */
void vko_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w,
                                  const int32_t* sorted_ids, float* out, int M, int width,
                                  int top_k, int EM) {
  const int N = M * top_k;
  for (int r = 0; r < EM; ++r) {
    const int flat = sorted_ids[r];
    if (flat < 0 || flat >= N) continue;
    const float w = topk_w[r];
    const float* src = partial + (size_t)r * width;
    float* dst = out + (size_t)(flat / top_k) * width;
    for (int j = 0; j < width; ++j) dst[j] += src[j] * w;
  }
}

/* moe_aux.cpp:290-321 */
void vko_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                    const float* topk_w, const int32_t* sorted_ids, float* out,
                                    int M, int width, int top_k, int EM, int group_size) {
  const int N = M * top_k;
  const int n_groups = width / group_size;
  for (int r = 0; r < EM; ++r) {
    const int flat = sorted_ids[r];
    if (flat < 0 || flat >= N) continue;
    const float w = topk_w[r];
    const uint8_t* pq = partial_q + (size_t)r * (width / 2);
    const uint8_t* ps = partial_s + (size_t)r * n_groups;
    float* dst = out + (size_t)(flat / top_k) * width;
    for (int g = 0; g < n_groups; ++g) {
      const float scale = aux_ue8m0_to_float(ps[g]);
      const int base = g * group_size;
      for (int i = 0; i < group_size; i += 2) {
        const float lo = fp4_nibble_to_float(pq[base / 2 + i / 2] & 0x0F) * scale;
        const float hi = fp4_nibble_to_float((pq[base / 2 + i / 2] >> 4) & 0x0F) * scale;
        dst[base + i] += lo * w;
        dst[base + i + 1] += hi * w;
      }
    }
  }
}

/* The activations a W4A4 layer multiplies: dequantised MXFP4 of one group of 32 bf16
 * values (exactly representable in bf16).  Used by the grouped GEMMs' operand model. */
void vko_aux_model_block32(const uint16_t* a, float* out) {
  uint8_t pk[16], sc[1];
  quant_row(a, pk, sc, 32, 32);
  const float scale = aux_ue8m0_to_float(sc[0]);
  for (int i = 0; i < 32; ++i) {
    const uint8_t nib = (i & 1) ? (uint8_t)(pk[i / 2] >> 4) : (uint8_t)(pk[i / 2] & 15);
    out[i] = fp4_nibble_to_float(nib) * scale;
  }
}
