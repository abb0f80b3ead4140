// moe_prefill.hip — the grouped GEMMs of the fused MXFP4 MoE layer for
// prefill-sized batches, on weights prepacked at load time.
//
//   stage 0  act[r, 0:I]  = bf16(act_fn(A[tok(r)] . W13[e, 0:I]^T + b13, A[tok(r)] . W13[e, I:2I]^T + b13))
//   stage 1  y[r, :]      = (act[r] . W2[e]^T + b2) * topk_w[flat(r)],  pos[flat(r)] = r
//
// (reference semantics: src/c/vkernels/kernels/moe_fused.cpp:235-564; the
// per-token sum of the y rows is combine_kernel's, in moe_gemm.hip.)
//
// Arithmetic.  v_mfma_scale_f32_32x32x64_f8f6f4 with the weights as the FP4
// (E2M1) operand and the activations as FP6 (E2M3) operands, both at the FP4
// rate of the matrix cores.  The weight codes are moved onto the OCP code
// points and their scale bytes decremented once, when the weights are
// prepacked (mxfp4.hpp: the reference's decode table is half of OCP's).  A
// bf16 activation is fed as a sum of TERMS FP6 terms per block of 32 along K:
//     t0 = Q(a / s0) s0,  t1 = Q((a - t0) / s1) s1,  t2 = Q((a - t0 - t1) / s2) s2,
// Q = round to nearest even on the E2M3 grid, s_i = 2^(e_i - 2 - 127) with e_i the
// largest exponent field of what the terms before left in the block (e_0: of the
// block itself); one MFMA per term, the term's scale byte being e_i - 2.  Three
// terms represent a bf16 value exactly unless it lies more than 2^-13 below the
// largest of its block; two terms leave an error of at most 2^-10 of the block's
// largest.  By default the first stage takes three terms and the second two
// (VK_HIP_MOE_SPLIT3 / VK_HIP_MOE_SPLIT2: three / two in both); TERMS = 1 is the
// W4A4 mode (MXFP4 activations, FP4 x FP4).
// Units whose weights hold an inf/NaN code or a scale byte outside
// [kScaleLo, kScaleHi] (flagged when the weights are prepacked) and segments
// with a row whose blocks are outside the representable range (flagged when
// the rows are split) are recomputed by exact_unit_mx: integer-exact
// dequantisation of the weights as the raw tensors hold them (read back from the
// prepacked form: a flagged unit keeps them there as they are, any other has
// the move onto the OCP points undone), bf16 MFMAs, bf16 rows from global memory.
//
// Work split.  A workgroup of 4 wavefronts (one per SIMD, 512 registers each)
// takes a window of 128 sorted rows -- cut into segments of consecutive blocks
// of one expert -- against 4 weight units; a unit is 128 weight rows (stage 0:
// 64 gate rows and the 64 up rows of the same columns, so the activation is
// fused; stage 1: 128 consecutive rows) = 4 MFMA tiles of 32, private to one
// wavefront: 4 x 4 accumulator tiles of 32 x 32 = 256 registers.  Per K step
// of 128:
//   * the split rows of the window (TERMS x 128 bytes per row) arrive in LDS
//     by the DMA form of the global load, two steps ahead, as whole cache
//     lines, the 16-byte pieces of a row rotated by the row index so that the
//     MFMA operand reads are conflict-free; shared by the four wavefronts, one
//     barrier per step;
//   * the wavefront's weights arrive straight in registers, two steps ahead:
//     the prepacked layout stores a unit's K step as 8 operand tiles of 64
//     lanes x 16 bytes in lane order, then 8 scale bytes per lane, 8704
//     contiguous bytes, so every load instruction reads 1 KiB contiguously;
//   * every operand read from LDS (32 bytes per lane: 24 of codes, the block's
//     scale byte, padding) feeds 4 MFMAs of 32 cycles; no vector arithmetic
//     sits between them.
// All loads are issued by inline assembly and waited for with counted
// s_waitcnt, because each wavefront issues them in a fixed order.
//
// Workgroup ids are mapped to (window, unit group) so that the 32 workgroups
// resident on one XCD at a time cover 4 windows x 8 unit groups or the like:
// the rows of a window and the weights of an expert are then fetched into
// that XCD's L2 once and shared.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "moe_common.hpp"
#include "moe_prefill_layout.hpp"
#include "vk_internal.hpp"

namespace vk {
namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(6))) uint32_t u32x6;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(32))) float f32x32;
typedef __attribute__((ext_vector_type(32))) __bf16 bf16x32;

struct MxArgs {
  const uint8_t* Wp;       // prepacked weights of the stage
  const uint8_t* Wflags;   // [E, units]: 1 = the unit takes the exact path
  const uint16_t* A;       // bf16 rows (exact path): stage 0 A [M, K], stage 1 act [EM, K]
  const uint8_t* Aq;       // split rows: row r = TERMS planes of Kp bytes at r * TERMS * Kp
  const uint8_t* row_bad;  // per row of Aq: 1 = outside the split's range
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const float* topk_w;
  const float* bias;
  uint16_t* act;           // stage 0 output [EM, ncols]
  float* y;                // stage 1 output [EM, ncols]
  int32_t* pos;            // stage 1: pos[flat] = sorted row
  float* preact;           // PREACT: the linear part alone, fp32 rows of 2 ncols (stage 0) / ncols (stage 1)
  int a_stride;            // elements between the bf16 rows of A (K, or the full width of a K slice)
  int n_flat, top_k, K, ncols, num_blocks, block_size;
  float swiglu_limit, beta, linear_beta;
  int activation;
  int units, col_groups, windows;
};

// ---------------------------------------------------------------------------
// Prepacking (load time).
// ---------------------------------------------------------------------------

// flags[e, unit] = 1 when a code of the unit's rows is inf/NaN or a scale byte
// lies outside [kScaleLo, kScaleHi].  One workgroup per (unit, expert).
__global__ __launch_bounds__(256) void prepack_flag_kernel(const uint8_t* __restrict__ W,
                                                           const uint8_t* __restrict__ Ws,
                                                           uint8_t* __restrict__ flags, int stage,
                                                           int rows_w, int ncols, int K, int units) {
  const int unit = blockIdx.x, e = blockIdx.y;
  const int n = threadIdx.x & 127, part = threadIdx.x >> 7;  // two threads per row
  const int row = mx_weight_row(stage, ncols, unit, n >> 5, n & 31);
  int bad = 0;
  if (row < rows_w) {
    const size_t r = (size_t)e * (size_t)rows_w + (size_t)row;
    const uint32_t* codes = reinterpret_cast<const uint32_t*>(W + r * (size_t)(K / 2));
    const uint8_t* sc = Ws + r * (size_t)(K / 32);
    uint32_t any = 0u;
    for (int i = part; i < K / 8; i += 2) any |= fp4x8_nonfinite(codes[i]);
    for (int g = part; g < K / 32; g += 2) any |= (uint32_t)(((uint32_t)sc[g] - kScaleLo) > (kScaleHi - kScaleLo));
    bad = any != 0u;
  }
  bad = __syncthreads_or(bad);
  if (threadIdx.x == 0) flags[(size_t)e * units + unit] = (uint8_t)(bad != 0);
}

// One workgroup per (K step, unit, expert): 512 pieces of 16 bytes (codes on the
// OCP points) and 64 x 8 scale bytes (decremented), zero codes / neutral scales
// where the unit or K is ragged.  A flagged unit keeps the codes and the scale bytes
// as they are in W / Ws: no fast path multiplies them, and the exact paths, which read
// the packed form as well, need the codes the move onto the OCP points would merge
// (the inf / NaN codes carry into the sign bit).
__global__ __launch_bounds__(256) void prepack_kernel(const uint8_t* __restrict__ W,
                                                      const uint8_t* __restrict__ Ws,
                                                      uint8_t* __restrict__ packed,
                                                      const uint8_t* __restrict__ flags, int stage,
                                                      int rows_w, int ncols, int K, int units,
                                                      int ksteps) {
  const int kstep = blockIdx.x, unit = blockIdx.y, e = blockIdx.z;
  const int groups = K / 32;
  const bool raw = flags[(size_t)e * units + unit] != 0;  // uniform
  uint8_t* dst = packed + mx_unit_offset(e, units, unit, ksteps) + (size_t)kstep * (size_t)kMxStepBytes;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int pc = threadIdx.x + 256 * i;  // [half][tile][lane]
    const int half = pc >> 8, t = (pc >> 6) & 3, lane = pc & 63;
    const int row = mx_weight_row(stage, ncols, unit, t, lane & 31);
    const int g = kstep * 4 + half * 2 + (lane >> 5);
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < rows_w && g < groups) {
      const size_t r = (size_t)e * (size_t)rows_w + (size_t)row;
      v = *reinterpret_cast<const u32x4*>(W + r * (size_t)(K / 2) + (size_t)g * 16);
      if (!raw) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = fp4x8_to_ocp_doubled(v[j]);
      }
    }
    *reinterpret_cast<u32x4*>(dst + (size_t)pc * 16) = v;
  }
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    uint32_t s8[2] = {0u, 0u};
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int row = mx_weight_row(stage, ncols, unit, t, lane & 31);
        const int g = kstep * 4 + half * 2 + (lane >> 5);
        uint32_t s = 127u;
        if (row < rows_w && g < groups)
          s = ((uint32_t)Ws[((size_t)e * (size_t)rows_w + (size_t)row) * (size_t)groups + g] - (raw ? 0u : 1u)) & 0xFFu;
        s8[half] |= s << (8 * t);
      }
    *reinterpret_cast<u32x2*>(dst + 8192 + lane * 8) = u32x2{s8[0], s8[1]};
  }
}

// ---------------------------------------------------------------------------
// bf16 rows [rows, K] -> split rows: per row TERMS planes of Kp bytes, a plane =
// Kp/32 blocks of 32 bytes: 24 bytes of FP6 codes (value i at bit 6 i), the
// term's scale byte, 7 zero bytes.  Blocks between K and Kp are zero with a
// neutral scale.  row_bad[r] = 1 when a block of the row is outside the range
// (inf/NaN, or a scale byte the scaled MFMA path does not take).
// One lane per block of 32; a workgroup takes as many whole rows as its 256 lanes hold
// (split_rows_per_group: 4 rows of 2048, 1 of 7168), so that short rows do not leave
// three of its four wavefronts idle.  With sorted_ids, x is in sorted order and only
// its routed rows (0 <= sorted_ids[r] < n_flat) are split: the padding rows of xq and
// row_bad keep what they held, and no consumer looks at them (a padding row of the
// alignment is most of the rows when experts are many and rows few).
// ---------------------------------------------------------------------------
__host__ __device__ constexpr int split_rows_per_group(int kp) { return kp / 32 >= 256 ? 1 : 256 / (kp / 32); }

// Workgroups of split_rows_fp6_kernel for `rows` rows of K values.
static inline dim3 split_grid(int rows, int K) {
  const int rpg = split_rows_per_group(mx_kp(K));
  return dim3((unsigned)((rows + rpg - 1) / rpg));
}

template <int TERMS>
__global__ __launch_bounds__(256) void split_rows_fp6_kernel(const uint16_t* __restrict__ x,
                                                             uint8_t* __restrict__ xq,
                                                             uint8_t* __restrict__ row_bad, int K,
                                                             int x_stride, int rows,
                                                             const int32_t* __restrict__ sorted_ids,
                                                             int n_flat, int32_t* __restrict__ fill,
                                                             int fill_n) {
  __shared__ int bad_rows[256];  // per row of the workgroup
  // (the second stage's table of sorted positions, set to "none" on the way: one launch less)
  for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < fill_n; i += (int)(gridDim.x * 256)) fill[i] = -1;
  const int kp = mx_kp(K);
  const int bpr = kp / 32;                       // blocks of a row
  const int rpg = split_rows_per_group(kp);      // rows of a workgroup
  const int sub = rpg > 1 ? (int)threadIdx.x / bpr : 0;  // this lane's row within the workgroup
  const size_t row = (size_t)blockIdx.x * rpg + sub;
  bool live = sub < rpg && row < (size_t)rows;
  if (live && sorted_ids != nullptr) {  // rows of a sorted order: only the routed ones are read
    const int f = sorted_ids[row];
    live = f >= 0 && f < n_flat;
  }
  if (threadIdx.x < rpg) bad_rows[threadIdx.x] = 0;
  __syncthreads();
  uint8_t* qrow = xq + row * (size_t)(TERMS * kp);
  int bad = 0;
  for (int b = rpg > 1 ? (int)threadIdx.x - sub * bpr : (int)threadIdx.x; live && b < bpr; b += 256) {
    union { u32x4 q[4]; bf16x32 v; uint32_t d[16]; } in;
#pragma unroll
    for (int i = 0; i < 4; ++i) in.q[i] = u32x4{0u, 0u, 0u, 0u};
    if (b * 32 < K) {
      const u32x4* src = reinterpret_cast<const u32x4*>(x + row * (size_t)x_stride + (size_t)b * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i) in.q[i] = src[i];
    }
    uint32_t emax = max(max(bf16x8_max_exponent(in.q[0]), bf16x8_max_exponent(in.q[1])),
                        max(bf16x8_max_exponent(in.q[2]), bf16x8_max_exponent(in.q[3])));
    uint32_t sb = emax - 2u;
    if (emax == 0u) {  // a block of zeros (or bf16 subnormals, taken as zero)
      sb = 127u;
    } else if (sb < kScaleLo + 4u * (TERMS - 1) || sb > kScaleHi) {
      bad = 1;
      sb = 127u;
    }
    f32x32 rest;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      rest[2 * i] = __uint_as_float(in.d[i] << 16);
      rest[2 * i + 1] = __uint_as_float(in.d[i] & 0xFFFF0000u);
    }
    uint32_t st = sb;
#pragma unroll
    for (int t = 0; t < TERMS; ++t) {
      union { bf16x32 v; uint32_t d[16]; u32x4 q[4]; } r16;  // the remainder is exact in bf16
#pragma unroll
      for (int i = 0; i < 16; ++i)
        r16.d[i] = (__float_as_uint(rest[2 * i]) >> 16) | (__float_as_uint(rest[2 * i + 1]) & 0xFFFF0000u);
      if (t > 0) {
        // a scale of the term's own, set as the first one's: from the largest exponent
        // field of what is left (at most 2^-4 of the previous term's scale, usually less:
        // then the term resolves a bit more), and not below the range of the path
        const uint32_t er = max(max(bf16x8_max_exponent(r16.q[0]), bf16x8_max_exponent(r16.q[1])),
                                max(bf16x8_max_exponent(r16.q[2]), bf16x8_max_exponent(r16.q[3])));
        st = er >= kScaleLo + 2u ? er - 2u : kScaleLo;
      }
      const float scale = __uint_as_float(st << 23);
      const u32x6 codes = __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(r16.v, scale);
      if (t + 1 < TERMS) rest -= __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(codes, scale);
      uint8_t* blk = qrow + (size_t)t * kp + (size_t)b * 32;
      *reinterpret_cast<u32x4*>(blk) = u32x4{codes[0], codes[1], codes[2], codes[3]};
      *reinterpret_cast<u32x4*>(blk + 16) = u32x4{codes[4], codes[5], st, 0u};
    }
  }
  if (bad != 0 && live) atomicOr(&bad_rows[sub], 1);
  __syncthreads();
  if (threadIdx.x < rpg && (size_t)blockIdx.x * rpg + threadIdx.x < (size_t)rows)
    row_bad[(size_t)blockIdx.x * rpg + threadIdx.x] = (uint8_t)(bad_rows[threadIdx.x] != 0);
}

// ---------------------------------------------------------------------------
// MXFP4 quantisation of activations, as the reference's mxfp4_moe_quant does
// (src/c/vkernels/kernels/moe_aux.cpp:99-139), per group of 32 bf16 values:
//   amax = the largest magnitude (a NaN never is, an inf is);
//   amax zero or non-finite: scale byte 0xFF and zero codes; else
//   scale byte s = clamp(ceil(log2(amax / 3)) + 127, 1, 254): with amax = 1.m x 2^x that
//   is the exponent field of amax, less one when m <= 1.5 (amax / 3 is a power of two
//   only for m = 1.5), at least 1;
//   code = nearest of {0, .25, 1, 1.5, 2, 3} to |a| / 2^(s-127), ties to the larger
//   (thresholds .125, .625, 1.25, 1.75, 2.5), sign bit set when a / scale < 0.
// d: the 32 values, two per dword; codes: 4 dwords, low nibble = even k.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void quant_group32(const uint32_t (&d)[16], uint32_t& sb, uint32_t (&codes)[4]) {
  // (bit patterns of non-negative floats order like the floats; a NaN counts as zero)
  uint32_t bits = 0u;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    uint32_t lo = d[i] & 0x7FFFu, hi = (d[i] >> 16) & 0x7FFFu;
    if (lo > 0x7F80u) lo = 0u;
    if (hi > 0x7F80u) hi = 0u;
    bits = max(bits, max(lo, hi));
  }
  const uint32_t ex = bits >> 7, mant = bits & 0x7Fu;
  if (ex == 0xFFu || bits == 0u) {
    sb = 0xFFu;
#pragma unroll
    for (int j = 0; j < 4; ++j) codes[j] = 0u;
    return;
  }
  int s = (int)ex - (mant <= 0x40u ? 1 : 0);
  if (ex == 0u || s < 1) s = 1;
  sb = (uint32_t)s;
  // a / 2^(s-127) as a product with 2^(127-s), exact (the rounding at underflow included)
  const float inv = s <= 253 ? __uint_as_float((uint32_t)(254 - s) << 23) : __uint_as_float(0x00400000u);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t word = 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t dw = d[j * 4 + (i >> 1)];
      const float a = __uint_as_float((i & 1) ? (dw & 0xFFFF0000u) : (dw << 16));
      const float x = __fmul_rn(a, inv);
      const float v = fabsf(x);
      uint32_t mag = 5u;              // also what a NaN gets: every comparison is false
      if (v < 0.125f) mag = 0u;
      else if (v < 0.625f) mag = 1u;
      else if (v < 1.25f) mag = 2u;
      else if (v < 1.75f) mag = 3u;
      else if (v < 2.5f) mag = 4u;
      if (x < 0.0f) mag |= 8u;
      word |= mag << (4 * i);
    }
    codes[j] = word;
  }
}

// Packed codes [rows, K/2] and scale bytes [rows, K/32] of bf16 rows: row r of the output
// is x[r] (sorted_ids null) or x[sorted_ids[r] / top_k], a padding row (id outside
// [0, n_flat)) giving zero codes and 0xFF scales (mxfp4_moe_sorted_quant,
// moe_aux.cpp:171-209).  One lane per group of 32.
__global__ __launch_bounds__(256) void mxfp4_quant_kernel(const uint16_t* __restrict__ x,
                                                          const int32_t* __restrict__ sorted_ids,
                                                          uint8_t* __restrict__ packed,
                                                          uint8_t* __restrict__ scales, int K,
                                                          int top_k, int n_flat) {
  const size_t row = blockIdx.x;
  const uint16_t* src = x + row * (size_t)K;
  bool pad = false;
  if (sorted_ids != nullptr) {
    const int flat = sorted_ids[row];
    pad = flat < 0 || flat >= n_flat;
    src = x + (size_t)(pad ? 0 : flat / top_k) * (size_t)K;
  }
  for (int g = threadIdx.x; g < K / 32; g += 256) {
    union { u32x4 q[4]; uint32_t d[16]; } in;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      in.q[i] = pad ? u32x4{0u, 0u, 0u, 0u} : reinterpret_cast<const u32x4*>(src + (size_t)g * 32)[i];
    uint32_t sb, codes[4];
    quant_group32(in.d, sb, codes);
    *reinterpret_cast<u32x4*>(packed + row * (size_t)(K / 2) + (size_t)g * 16) =
        u32x4{codes[0], codes[1], codes[2], codes[3]};
    scales[row * (size_t)(K / 32) + g] = (uint8_t)sb;
  }
}

// The same quantisation as the split rows of the W4A4 mode: one plane of Kp bytes per
// row, a block = the 32 codes moved onto the OCP code points (16 bytes), the scale byte
// less one, 15 zero bytes; zero groups get a neutral scale.  row_bad[r] = 1 when a scale
// byte is outside the range the scaled MFMA path takes.
__global__ __launch_bounds__(256) void quant_rows_w4_kernel(const uint16_t* __restrict__ x,
                                                            uint8_t* __restrict__ xq,
                                                            uint8_t* __restrict__ row_bad, int K,
                                                            const int32_t* __restrict__ sorted_ids,
                                                            int n_flat, int32_t* __restrict__ fill,
                                                            int fill_n) {
  for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < fill_n; i += (int)(gridDim.x * 256)) fill[i] = -1;
  const int kp = mx_kp(K);
  const size_t row = blockIdx.x;
  if (sorted_ids != nullptr) {  // as split_rows_fp6_kernel: routed rows only (uniform per workgroup)
    const int f = sorted_ids[row];
    if (f < 0 || f >= n_flat) return;
  }
  uint8_t* qrow = xq + row * (size_t)kp;
  int bad = 0;
  for (int b = threadIdx.x; b < kp / 32; b += 256) {
    union { u32x4 q[4]; uint32_t d[16]; } in;
#pragma unroll
    for (int i = 0; i < 4; ++i) in.q[i] = u32x4{0u, 0u, 0u, 0u};
    if (b * 32 < K) {
      const u32x4* src = reinterpret_cast<const u32x4*>(x + row * (size_t)K + (size_t)b * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i) in.q[i] = src[i];
    }
    uint32_t sb, codes[4];
    quant_group32(in.d, sb, codes);
    uint32_t st = 127u;
    if (sb != 0xFFu) {
      st = sb - 1u;
      if (st < kScaleLo || st > kScaleHi) bad = 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) codes[j] = fp4x8_to_ocp_doubled(codes[j]);
    }
    uint8_t* blk = qrow + (size_t)b * 32;
    *reinterpret_cast<u32x4*>(blk) = u32x4{codes[0], codes[1], codes[2], codes[3]};
    *reinterpret_cast<u32x4*>(blk + 16) = u32x4{st, 0u, 0u, 0u};
  }
  bad = __syncthreads_or(bad);
  if (threadIdx.x == 0) row_bad[row] = (uint8_t)(bad != 0);
}

// ---------------------------------------------------------------------------
// Exact path of one unit for the 32 rows of one row tile: acc[t] = C[weight row of
// tile t][activation row lane % 32] in the accumulator layout of the 32 x 32 MFMAs.
// a_row: the bf16 row of this lane's activation row, or null for a padding row.
// q_row (W4A4 mode): the row's quantised plane instead; its values are decoded exactly.
template <int STAGE>
__device__ __forceinline__ void exact_unit_mx(const MxArgs& p, int e, int unit, bool w_raw, const uint16_t* a_row,
                                              const uint8_t* q_row, int lane, f32x16 (&acc)[4]) {
  // The weights come from the packed form: K block g of row n of tile t is the 16 bytes
  // at step g / 4, half (g / 2) % 2, lane (g % 2, n) of the tile, its scale byte the one
  // for (half, t) of that lane's eight.  A flagged unit (w_raw) holds the codes and
  // scale bytes of the raw tensors; any other the codes moved onto the OCP points and
  // the scale bytes less one, both undone here (all its codes are finite).
  const int n = lane & 31, hh = lane >> 5;
  const int K = p.K;
  const int nsteps = mx_kp(K) / 128;
  const uint8_t* const ub = p.Wp + mx_unit_offset(e, p.units, unit, nsteps);
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
#pragma unroll 1
  for (int s = 0; s < K / 16; ++s) {  // 16 values of K: lane half hh takes 8 of them
    const int k = 16 * s + 8 * hh;
    u32x4 av = {0u, 0u, 0u, 0u};
    if (a_row != nullptr) av = *reinterpret_cast<const u32x4*>(a_row + k);
    if (q_row != nullptr) {  // 8 codes of block k / 32 back on the reference's code points
      const uint8_t* blk = q_row + (size_t)(k >> 5) * 32;
      uint32_t c = *reinterpret_cast<const uint32_t*>(blk + ((k & 31) >> 1));
      c -= (c & 0x44444444u) >> 1;
      av = dequant8_exact(c, ((uint32_t)blk[16] + 1u) & 0xFFu);
    }
    const int g = k >> 5;
    const uint8_t* const sb = ub + (size_t)(g >> 2) * kMxStepBytes;
    const int half = (g >> 1) & 1, lane_p = (g & 1) * 32 + n;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      uint32_t c = *reinterpret_cast<const uint32_t*>(sb + half * 4096 + t * 1024 + lane_p * 16 + ((k & 31) >> 1));
      uint32_t sc = sb[8192 + lane_p * 8 + half * 4 + t];
      if (!w_raw) {
        c -= (c & 0x44444444u) >> 1;
        sc = (sc + 1u) & 0xFFu;
      }
      const u32x4 wv = dequant8_exact(c, sc);
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(wv), as_bf16x8(av), acc[t], 0, 0, 0);
    }
  }
}

// Register load of 16 (8) bytes per lane at base + voff (+ an immediate), not
// waited for: the caller counts it and passes the registers through wait_loads.
template <int OFF>
__device__ __forceinline__ void load16_nowait(u32x4& dst, uint32_t voff, const uint8_t* base) {
  __asm__ volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(dst) : "v"(voff), "s"(base), "n"(OFF) : "memory");
}
__device__ __forceinline__ void load8_nowait(u32x2& dst, uint32_t voff, const uint8_t* base) {
  __asm__ volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(dst) : "v"(voff), "s"(base) : "memory");
}
// The DMA form with a uniform base and a 32-bit offset per lane: 16 bytes per lane to
// LDS at lds_base + 16 * lane.
__device__ __forceinline__ void dma16_saddr(uint32_t voff, const uint8_t* base, uint32_t lds_base) {
  __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voff), "s"(base)
                   : "memory");
}

struct WeightStep {  // one K step of a unit in registers
  u32x4 w[8];        // [half][tile]
  u32x2 sc;          // per lane: the 4 tiles' scale bytes of half 0, of half 1
};

// Waits until at most N vector-memory operations are outstanding; the registers of
// `ws` are operands so that no use of them moves above the wait.
template <int N>
__device__ __forceinline__ void wait_loads(WeightStep& ws) {
  __asm__ volatile("s_waitcnt vmcnt(%[n])"
                   : "+v"(ws.w[0]), "+v"(ws.w[1]), "+v"(ws.w[2]), "+v"(ws.w[3]), "+v"(ws.w[4]),
                     "+v"(ws.w[5]), "+v"(ws.w[6]), "+v"(ws.w[7]), "+v"(ws.sc)
                   : [n] "n"(N)
                   : "memory");
}

// The same, and for the wavefront's LDS reads as well.
template <int N>
__device__ __forceinline__ void wait_loads_and_reads(WeightStep& ws) {
  __asm__ volatile("s_waitcnt vmcnt(%[n]) lgkmcnt(0)"
                   : "+v"(ws.w[0]), "+v"(ws.w[1]), "+v"(ws.w[2]), "+v"(ws.w[3]), "+v"(ws.w[4]),
                     "+v"(ws.w[5]), "+v"(ws.w[6]), "+v"(ws.w[7]), "+v"(ws.sc)
                   : [n] "n"(N)
                   : "memory");
}

__device__ __forceinline__ i32x8 fp4_operand_ocp(u32x4 w) {  // codes already on the OCP points
  const i32x4 y = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  return __builtin_shufflevector(y, y, 0, 1, 2, 3, -1, -1, -1, -1);
}

// One scaled MFMA: A = FP4 (cbsz 4) with scale byte T of wscale.  B = the operand read
// from LDS: FP6 E2M3 (blgp 2, scale in byte 0 of b[6]) or, in the W4A4 mode, FP4 (blgp 4,
// codes in b[0..3], scale in byte 0 of b[4]).
template <int T, bool W4A4>
__device__ __forceinline__ f32x16 mfma_fp4_act(u32x4 w, i32x8 b, f32x16 acc, uint32_t wscale) {
  if constexpr (W4A4)
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fp4_operand_ocp(w), b, acc, 4, 4, T,
                                                           (int)wscale, 0, b[4]);
  else
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fp4_operand_ocp(w), b, acc, 4, 2, T,
                                                           (int)wscale, 0, b[6]);
}

// PREACT: the stage's linear part alone (tensor-parallel callers sum it over their K slices
// before the epilogue): the accumulators of the routed rows go to p.preact as fp32, no
// bias, no activation, no routing weight; rows that are not routed are left as they are.
template <int STAGE, int TERMS, bool PREACT = false>
__global__ __launch_bounds__(64 * kMxWaves) void tile_mx_kernel(MxArgs p) {
  constexpr int R = kMxRing;
  constexpr int kSlotBytes = kMxRows * TERMS * 128;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  extern __shared__ u32x4 mx_lds[];
  __shared__ int win_flat[kMxRows];  // sorted_ids of the window's rows, asked for before its experts are known
  __shared__ int row_flat[kMxRows];
  __shared__ float row_w[kMxRows];  // stage 1: the routing weight of every row (0 where none is routed)
  __shared__ int seg_hi[2];   // highest routed row index among rows 0..63 / 64..127 (or -1)
  __shared__ int seg_bad[2];  // a routed row of the half is outside the split's range

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31;
  const int hh = lane >> 5;

  // ---- (window, unit group) of this workgroup: chunks of 32 consecutive tiles go to
  // one XCD (workgroup ids go round-robin over the 8 XCDs), chunk after chunk ----
  const int total = p.col_groups * p.windows;
  const int slot = blockIdx.x >> 3;
  const int logical = ((slot >> 5) * 8 + (blockIdx.x & 7)) * 32 + (slot & 31);
  if (logical >= total) return;
  const int window = logical / p.col_groups;
  const int colg = logical - window * p.col_groups;

  const int K = p.K;
  const int Kp = mx_kp(K);
  const int nsteps = Kp / 128;
  const int unit_raw = colg * kMxWaves + wave;
  const bool has_unit = unit_raw < p.units;
  const int unit = has_unit ? unit_raw : 0;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr)mx_lds;
  const uint8_t* lds_bytes = reinterpret_cast<const uint8_t*>(mx_lds);

  // Vector-memory operations of a wavefront per K step (for step c + 2): 4 TERMS row
  // copies, 8 weight loads, 1 scale load.
  constexpr int kRowOps = mx_row_ops(TERMS);
  constexpr int kOps = mx_step_ops(TERMS);

  // the rows of this workgroup's window
  const int total_rows = p.num_blocks * p.block_size;
  const int win = mx_window_rows(p.block_size);
  const int win_end = min(window * win + win, total_rows);

  auto segment = [&](const int row0_, const int n_rows_, const int e_) {
    // uniform by construction; said so, so that addresses built on them stay scalar
    const int row0 = __builtin_amdgcn_readfirstlane(row0_);
    const int n_rows = __builtin_amdgcn_readfirstlane(n_rows_);
    const int e = __builtin_amdgcn_readfirstlane(e_);
    __syncthreads();  // the previous segment is done with row_flat and the ring (and win_flat is written)
    // The ids of the segment's rows come from the window's, already in LDS.  What hangs on an
    // id -- the row's flag of the split and, in the second stage, its routing weight -- is
    // asked for here and looked at behind the K loop: only the epilogue needs it, and a
    // round trip to memory in front of the first row copy is a microsecond of every workgroup.
    int bad_v = 0;
    float w_v = 0.f;
    if (tid < kMxRows) {
      int f = -1;
      if (tid < n_rows) {
        f = win_flat[row0 - window * win + tid];
        if (f < 0 || f >= p.n_flat) f = -1;
      }
      row_flat[tid] = f;
      if (f >= 0) bad_v = p.row_bad[STAGE == 0 ? f / p.top_k : row0 + tid];
      if (STAGE == 1 && !PREACT && f >= 0) w_v = p.topk_w[f];
      const unsigned long long routed = __ballot(f >= 0);
      if (lane == 0) seg_hi[wave] = routed != 0ull ? 63 - (int)__builtin_clzll(routed) : -1;
    }
    // A barrier for LDS alone: __syncthreads() would also wait for the two loads just
    // asked for (a workgroup-wide fence makes every memory operation of the wavefront land).
    __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const int hi = seg_hi[1] >= 0 ? 64 + seg_hi[1] : seg_hi[0];
    const int n_live = (hi + 32) >> 5;  // row tiles of 32 up to the last routed row
    if (n_live == 0) return;            // uniform
    const bool w_slow = has_unit && p.Wflags[(size_t)e * p.units + unit] != 0;  // uniform per wavefront

    // ---- row copies: one instruction moves 8 rows x 128 bytes of one term.  Lane
    // (r, c) = (lane / 8, lane % 8) copies piece c ^ r of its row, so LDS position c of
    // row r holds piece c ^ (r & 7).  Wavefront w copies row tile w (32 rows).
    uint32_t cp_off[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int r = lane >> 3, c = lane & 7;
      const int rl = wave * 32 + g * 8 + r;
      const int f = row_flat[rl];
      size_t grow;
      if (STAGE == 0) grow = f >= 0 ? (size_t)(f / p.top_k) : 0;
      else grow = rl < n_rows ? (size_t)(row0 + rl) : (size_t)row0;
      cp_off[g] = mx_row_copy_lane_offset(grow, TERMS, Kp, lane);
    }
    auto copy_rows = [&](int step, int d) {  // operation d (0 .. 4 TERMS - 1) of the step's row copies
      const int term = d >> 2, g = d & 3;
      // (past the end: the last step again)
      dma16_saddr(cp_off[g] + mx_row_copy_step_offset(term, Kp, step, nsteps), p.Aq,
                  lds_base + mx_row_copy_lds(step, wave, TERMS, term, g));
    };
    // ---- weight loads
    const uint8_t* wp_unit = p.Wp + mx_unit_offset(e, p.units, unit, nsteps);
    const uint32_t voff16 = (uint32_t)lane * 16u, voff8 = (uint32_t)lane * 8u;
    auto load_weights = [&](WeightStep& ws, int step, int j) {  // operation j (0 .. 8)
      const uint8_t* base = wp_unit + mx_step_offset(step, nsteps);
      // (the immediates and lane offsets below are mx_weight_load_offset(j, lane))
      static_assert(mx_weight_load_offset(3, 2) == 3072 + 32 && mx_weight_load_offset(6, 0) == 4096 + 2048 &&
                        mx_weight_load_offset(8, 3) == 8192 + 24,
                    "weight loads and their layout function disagree");
      switch (j) {
        case 0: load16_nowait<0>(ws.w[0], voff16, base); break;
        case 1: load16_nowait<1024>(ws.w[1], voff16, base); break;
        case 2: load16_nowait<2048>(ws.w[2], voff16, base); break;
        case 3: load16_nowait<3072>(ws.w[3], voff16, base); break;
        case 4: load16_nowait<0>(ws.w[4], voff16, base + 4096); break;
        case 5: load16_nowait<1024>(ws.w[5], voff16, base + 4096); break;
        case 6: load16_nowait<2048>(ws.w[6], voff16, base + 4096); break;
        case 7: load16_nowait<3072>(ws.w[7], voff16, base + 4096); break;
        default: load8_nowait(ws.sc, voff8, base + 8192); break;
      }
    };
    // operation k (0 .. kOps - 1) of what a K step issues for step `step`
    auto issue = [&](WeightStep& ws, int step, int k) {
      if (k < kRowOps) copy_rows(step, k);
      else load_weights(ws, step, k - kRowOps);
    };

    // ---- operand reads: lane (ln, hh) takes block 2 half + hh of row ln of row tile m:
    // pieces 2 blk and 2 blk + 1, at positions (2 blk) ^ (ln & 7) and that ^ 1.  The four
    // lane-dependent offsets (half 0 / 1, first / second piece) are added to the slot's
    // base once per K step; row tile and term are immediate offsets of the reads.
    uint32_t rd_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) rd_off[j] = mx_operand_lane_offset(j, ln, hh);
    struct SlotBase {
      const uint8_t* b[4];
    };
    auto slot_base = [&](int slot_) {
      SlotBase sb;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t off = rd_off[j] + mx_operand_tile_offset(slot_, TERMS, 0, 0);
        __asm__ volatile("" : "+v"(off));  // one register per base: nothing to precompute per tile
        sb.b[j] = lds_bytes + off;
      }
      return sb;
    };
    auto read_operand = [&](const SlotBase& sb, int m, int term, int half) {
      const int tile_off = (int)mx_operand_tile_offset(0, TERMS, m, term);
      const u32x4 lo = *reinterpret_cast<const u32x4*>(sb.b[2 * half] + tile_off);
      const u32x4 hi4 = *reinterpret_cast<const u32x4*>(sb.b[2 * half + 1] + tile_off);
      return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                   (int)hi4[0], (int)hi4[1], (int)hi4[2], (int)hi4[3]};
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[m][t][i] = 0.f;

    // The K loop, compiled once per number of live row tiles.  A step is Q groups of 4
    // MFMAs (one operand of rows against the 4 weight tiles).  Software pipeline over the
    // groups: while group q multiplies, the operand of group q + 1 is completed and the
    // reads of group q + 2 are issued, across the step boundary as well, so the matrix pipe
    // never waits for LDS.  Memory operations for step c + 2 are issued in groups 0 .. Q-3
    // of step c.  After group Q-3 comes the step's one barrier: each wavefront has waited
    // for its loads of step c + 1 (only the kOps operations of this step may be
    // outstanding) and for its LDS reads of step c (all issued by then), so behind the
    // barrier step c + 1 can be read and the slot of step c can take step c + 3.
    auto k_loop = [&](auto live_c) {
      constexpr int LIVE = decltype(live_c)::value;
      constexpr int Q = mx_step_groups(LIVE, TERMS);       // groups (operand reads) per step
      constexpr int kPer = mx_ops_per_group(LIVE, TERMS);  // memory operations per issuing group
      static_assert(Q >= 4 && kPer * (Q - 2) >= kOps, "a step's loads are all issued before its wait");
      auto group_operand = [&](const SlotBase& sb, int q) {
        return read_operand(sb, (q / TERMS) % LIVE, q % TERMS, q / (LIVE * TERMS));
      };
      WeightStep ws[3];
      // prologue: the loads of steps 0 and 1; step 0's have landed in every wavefront
      // once only step 1's are outstanding
#pragma unroll
      for (int k = 0; k < kOps; ++k) issue(ws[0], 0, k);
#pragma unroll
      for (int k = 0; k < kOps; ++k) issue(ws[1], 1, k);
      wait_loads<kOps>(ws[0]);
      __builtin_amdgcn_s_barrier();
      __asm__ volatile("" ::: "memory");
      SlotBase sb = slot_base(0);
      i32x8 cur = group_operand(sb, 0);
      i32x8 nxt = group_operand(sb, 1);

      // one K step; i = c % 3 picks the register set of the step's weights
      auto step = [&](auto i_c, const int c) {
        constexpr int i = decltype(i_c)::value;
        constexpr int in1 = (i + 1) % 3, in2 = (i + 2) % 3;
        int slot_next = mx_ring_slot(c + 1);
        __asm__ volatile("" : "+s"(slot_next));
        const SlotBase sbn = slot_base(slot_next);
        int issued = 0;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
          const int half = q / (LIVE * TERMS), m = (q / TERMS) % LIVE;
          const uint32_t wsc = ws[i].sc[half];
          // (a wavefront without a unit multiplies unit 0's weights and drops the result)
          acc[m][0] = mfma_fp4_act<0, TERMS == 1>(ws[i].w[half * 4 + 0], cur, acc[m][0], wsc);
          __builtin_amdgcn_sched_barrier(0);
          // reads of group q + 2; the last two groups read the next step's first two
          const i32x8 pend = q + 2 < Q ? group_operand(sb, q + 2) : group_operand(sbn, q + 2 - Q);
          __builtin_amdgcn_sched_barrier(0);
          acc[m][1] = mfma_fp4_act<1, TERMS == 1>(ws[i].w[half * 4 + 1], cur, acc[m][1], wsc);
          __builtin_amdgcn_sched_barrier(0);
          if (q < Q - 2) {
#pragma unroll
            for (int k = 0; k < kPer; ++k)
              if (issued + k < kOps) issue(ws[in2], c + 2, issued + k);
            issued += kPer;
          }
          __builtin_amdgcn_sched_barrier(0);
          acc[m][2] = mfma_fp4_act<2, TERMS == 1>(ws[i].w[half * 4 + 2], cur, acc[m][2], wsc);
          __builtin_amdgcn_sched_barrier(0);
          __asm__ volatile("" : "+v"(nxt));  // complete from here on (read a group ago)
          __builtin_amdgcn_sched_barrier(0);
          acc[m][3] = mfma_fp4_act<3, TERMS == 1>(ws[i].w[half * 4 + 3], cur, acc[m][3], wsc);
          __builtin_amdgcn_sched_barrier(0);
          if (q == mx_wait_group(LIVE, TERMS)) {
            wait_loads_and_reads<kOps>(ws[in1]);
            __builtin_amdgcn_s_barrier();
            __asm__ volatile("" ::: "memory");
          }
          cur = nxt;
          nxt = pend;
        }
        sb = sbn;
      };
      // three steps per pass of the loop body (no exit inside it), then the remainder
      int c0 = 0;
#pragma unroll 1
      for (; c0 + 3 <= nsteps; c0 += 3) {
        step(IntC<0>{}, c0);
        step(IntC<1>{}, c0 + 1);
        step(IntC<2>{}, c0 + 2);
      }
      if (c0 < nsteps) step(IntC<0>{}, c0);
      if (c0 + 1 < nsteps) step(IntC<1>{}, c0 + 1);
      // the loads issued past the last step write registers and the ring: let them land
      wait_loads<0>(ws[0]);
      wait_loads<0>(ws[1]);
      wait_loads<0>(ws[2]);
    };
    // (one plane per row: a step of one row tile would be shorter than the pipeline)
    if (n_live > 3) k_loop(IntC<4>{});
    else if (n_live == 3) k_loop(IntC<3>{});
    else if (n_live == 2 || TERMS == 1) k_loop(IntC<2>{});
    else if constexpr (TERMS > 1) k_loop(IntC<1>{});
    if (tid < kMxRows) {  // (wavefronts 0 and 1: whole wavefronts)
      if (STAGE == 1 && !PREACT) row_w[tid] = w_v;
      const unsigned long long any_bad = __ballot(bad_v != 0);
      if (lane == 0) seg_bad[wave] = any_bad != 0ull;
    }
    __syncthreads();
    const bool slow = (seg_bad[0] | seg_bad[1]) != 0 || w_slow;

    if (STAGE == 1 && !PREACT && colg == 0 && tid < n_rows && row_flat[tid] >= 0) p.pos[row_flat[tid]] = row0 + tid;
    if (!has_unit) return;

    // ---- epilogue: lane (ln, hh) holds, of activation row 32 m + ln, the weight rows
    // 8 (i / 4) + 4 hh + i % 4 of each tile: a few columns of 32 different rows.  Stored
    // like that, every store instruction touches 64 cache lines; instead the values of 32
    // rows go through a staging area of the wavefront's own in the ring (free after the
    // barrier above) and leave as whole lines: 4 rows x 256 bytes (8 rows x 128 bytes in
    // stage 0) per store instruction ----
    uint8_t* stage_lds = reinterpret_cast<uint8_t*>(mx_lds) + mx_stage_base(wave, TERMS);
    auto wave_fence = [] {  // LDS operations of a wavefront execute in order; this keeps the compiler's too
      __asm__ volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // The biases of the columns this lane holds (the same for every row tile), tile by
    // tile as the accumulators are laid out: asked for here, all at once, not value by
    // value inside the loops below.
    const bool has_bias = !PREACT && p.bias != nullptr;  // uniform
    f32x4 bias_v[4][4];  // [tile][row group]
    if (has_bias) {
      // stage 0: tiles 0, 1 = gate columns, 2, 3 = the same columns of up
      // stage 1: the last unit may be ragged (ncols is a multiple of 64); its columns past
      // the end are not stored, so the first tiles' biases stand in
      const float* b = p.bias + (STAGE == 0 ? (size_t)e * (size_t)(2 * p.ncols) + unit * 64
                                            : (size_t)e * (size_t)p.ncols + unit * kMxUnitRows) + hh * 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int c = STAGE == 0 ? (t >> 1) * p.ncols + (t & 1) * 32
                                 : (unit * kMxUnitRows + (t >> 1) * 64 < p.ncols ? t * 32 : 0);
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) bias_v[t][rg] = *reinterpret_cast<const f32x4u*>(b + c + rg * 8);
      }
    } else if (STAGE == 0 && !PREACT && p.activation == 1) {  // the one loop that adds them without a bias
#pragma unroll
      for (int i = 0; i < 16; ++i) bias_v[i >> 2][i & 3] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      if (m >= n_live) break;
      f32x16 (&tile)[4] = acc[m];
      const int flat = row_flat[m * 32 + ln];
      const int srow = row0 + m * 32 + ln;
      const unsigned long long routed = __ballot(flat >= 0);  // bit r (< 32): row 32 m + r is routed
      if (slow) {
        const uint16_t* a_row = nullptr;
        const uint8_t* q_row = nullptr;
        if (flat >= 0) {
          const size_t grow = (size_t)(STAGE == 0 ? flat / p.top_k : srow);
          if (TERMS == 1) q_row = p.Aq + grow * (size_t)Kp;
          else a_row = p.A + grow * (size_t)p.a_stride;
        }
        exact_unit_mx<STAGE>(p, e, unit, w_slow, a_row, q_row, lane, tile);
      }
      if constexpr (PREACT) {
        // the accumulators as they are: 64 columns (two tiles) at a time through the
        // wavefront's staging area, whole lines out, routed rows only
        constexpr int kPitch = kMxYPitch;
        const int width = STAGE == 0 ? 2 * p.ncols : p.ncols;
#pragma unroll
        for (int tp = 0; tp < 2; ++tp) {
          // stage 0: tiles 0, 1 = gate columns of the unit, 2, 3 = the same columns of up
          const int col0 = STAGE == 0 ? tp * p.ncols + unit * 64 : unit * kMxUnitRows + tp * 64;
          if (STAGE == 1 && col0 >= p.ncols) break;  // uniform: the last unit may be ragged
#pragma unroll
          for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
              const int t = 2 * tp + tl;
              const int cl = tl * 32 + rg * 8 + hh * 4;
              *reinterpret_cast<f32x4*>(stage_lds + ln * kPitch + cl * 4) =
                  f32x4{tile[t][rg * 4], tile[t][rg * 4 + 1], tile[t][rg * 4 + 2], tile[t][rg * 4 + 3]};
            }
          wave_fence();
          f32x4 v[8];
#pragma unroll
          for (int pass = 0; pass < 8; ++pass)
            v[pass] = *reinterpret_cast<const f32x4*>(stage_lds + (pass * 4 + (lane >> 4)) * kPitch + (lane & 15) * 16);
          wave_fence();
          float* dst = p.preact + (size_t)(row0 + m * 32 + (lane >> 4)) * (size_t)width + col0 + (lane & 15) * 4;
#pragma unroll
          for (int pass = 0; pass < 8; ++pass) {
            if ((routed >> (pass * 4 + (lane >> 4))) & 1ull) *reinterpret_cast<f32x4*>(dst) = v[pass];
            dst += 4 * (size_t)width;
          }
        }
      } else if (STAGE == 0) {
        constexpr int kPitch = kMxActPitch;
        // 128 activation values per lane and row tile.  A wavefront runs alone on its SIMD,
        // so a branch per value (bias or not, clamp or not, which activation) is paid in
        // full: the loop is compiled once per combination of what is uniform, act_value's
        // formulas with their parameters known at compile time.
        auto act_rows = [&](auto bias_c, auto limit_c, auto situ_c) {
          constexpr bool kBias = decltype(bias_c)::value != 0, kLimit = decltype(limit_c)::value != 0,
                         kSitu = decltype(situ_c)::value != 0;
          float limit = 0.0f, beta = 0.0f, linear_beta = 0.0f, inv_beta = 0.0f, inv_linear_beta = 0.0f;
          if constexpr (kLimit) limit = p.swiglu_limit > 0.0f ? p.swiglu_limit : __builtin_inff();
          if constexpr (kSitu) {
            beta = p.beta;
            linear_beta = p.linear_beta;
            inv_beta = __builtin_amdgcn_rcpf(beta);
            inv_linear_beta = linear_beta > 0.0f ? __builtin_amdgcn_rcpf(linear_beta) : 0.0f;
          }
#pragma unroll
          for (int tp = 0; tp < 2; ++tp)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
              const int cl = tp * 32 + rg * 8 + hh * 4;  // column within the unit's 64
              uint32_t packed[2];
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                float g = tile[tp][rg * 4 + i], u = tile[tp + 2][rg * 4 + i];
                if constexpr (kBias) {
                  g += bias_v[tp][rg][i];
                  u += bias_v[tp + 2][rg][i];
                }
                float a;
                if constexpr (kSitu) {
                  a = situ_value(g, u, beta, inv_beta, linear_beta, inv_linear_beta);
                } else {
                  if constexpr (kLimit) {
                    g = g > limit ? limit : g;  // (a NaN stays one, as in act_value)
                    u = u > limit ? limit : u;
                    u = u < -limit ? -limit : u;
                  }
                  a = act_value(0, g, u, 0.0f, 0.0f, 0.0f);
                }
                const uint32_t v = f32_to_bf16_bits(a);
                if (i & 1) packed[i >> 1] |= v << 16;
                else packed[i >> 1] = v;
              }
              *reinterpret_cast<uint2*>(stage_lds + ln * kPitch + cl * 2) = make_uint2(packed[0], packed[1]);
            }
        };
        if (flat >= 0) {
          // (uniform conditions.  Four loops, not eight: a clamp that is off is a clamp at
          // infinity, and SiTU without biases adds zeros)
          const bool clamp = p.swiglu_limit > 0.0f;
          if (p.activation == 1) act_rows(IntC<1>{}, IntC<0>{}, IntC<1>{});
          else if (has_bias) act_rows(IntC<1>{}, IntC<1>{}, IntC<0>{});
          else if (clamp) act_rows(IntC<0>{}, IntC<1>{}, IntC<0>{});
          else act_rows(IntC<0>{}, IntC<0>{}, IntC<0>{});
        }
        wave_fence();
        u32x4 v[4];  // all the reads, one wait, then the stores: 8 rows x 128 bytes per instruction
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
          v[pass] = *reinterpret_cast<const u32x4*>(stage_lds + (pass * 8 + (lane >> 3)) * kPitch + (lane & 7) * 16);
        wave_fence();
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
          const int r = pass * 8 + (lane >> 3), piece = lane & 7;
          if ((routed >> r) & 1ull)
            *reinterpret_cast<u32x4*>(p.act + (size_t)(row0 + m * 32 + r) * (size_t)p.ncols + unit * 64 +
                                      piece * 8) = v[pass];
        }
      } else {
        // A wavefront runs alone on its SIMD, so every branch and every predicate of this
        // code is paid in full; it is therefore specialised, per row tile, on what is
        // uniform: a bias or none, and whether the tile's 32 rows all belong to this
        // workgroup's window.  Then rows that are not routed are stored like the others
        // (with a routing weight of zero): nothing reads them (pos never points at them),
        // and a later segment of this window, if they are its rows, overwrites them.
        constexpr int kPitch = kMxYPitch;
        // (from LDS, put there when the rows were listed: a load from memory still pending
        // when the stores begin makes every later wait for it a wait for those stores)
        const float w = row_w[m * 32 + ln];
        auto store_rows = [&](auto bias_c, auto guard_c) {
          constexpr bool kBias = decltype(bias_c)::value != 0, kGuard = decltype(guard_c)::value != 0;
#pragma unroll
          for (int tp = 0; tp < 2; ++tp) {  // tiles 2 tp, 2 tp + 1: 64 columns
            const int col0 = unit * kMxUnitRows + tp * 64;
            if (col0 >= p.ncols) break;  // uniform: the last unit may be ragged (ncols is a multiple of 64)
#pragma unroll
            for (int tl = 0; tl < 2; ++tl)
#pragma unroll
              for (int rg = 0; rg < 4; ++rg) {
                const int t = 2 * tp + tl;
                const int cl = tl * 32 + rg * 8 + hh * 4;
                f32x4 v = {tile[t][rg * 4], tile[t][rg * 4 + 1], tile[t][rg * 4 + 2], tile[t][rg * 4 + 3]};
                if constexpr (kBias) v += bias_v[t][rg];
                *reinterpret_cast<f32x4*>(stage_lds + ln * kPitch + cl * 4) = v * w;
              }
            wave_fence();
            f32x4 v[8];  // all the reads, one wait, then the stores: 4 rows x 256 bytes per instruction
#pragma unroll
            for (int pass = 0; pass < 8; ++pass)
              v[pass] = *reinterpret_cast<const f32x4*>(stage_lds + (pass * 4 + (lane >> 4)) * kPitch + (lane & 15) * 16);
            wave_fence();
            float* dst = p.y + (size_t)(row0 + m * 32 + (lane >> 4)) * (size_t)p.ncols + col0 + (lane & 15) * 4;
#pragma unroll
            for (int pass = 0; pass < 8; ++pass) {
              if constexpr (kGuard) {
                if ((routed >> (pass * 4 + (lane >> 4))) & 1ull) *reinterpret_cast<f32x4*>(dst) = v[pass];
              } else {
                *reinterpret_cast<f32x4*>(dst) = v[pass];
              }
              dst += 4 * (size_t)p.ncols;
            }
          }
        };
        const bool inside = row0 + m * 32 + 32 <= win_end;  // uniform
        if (!has_bias) {
          if (inside) store_rows(IntC<0>{}, IntC<0>{});
          else store_rows(IntC<0>{}, IntC<1>{});
        } else {
          if (inside) store_rows(IntC<1>{}, IntC<0>{});
          else store_rows(IntC<1>{}, IntC<1>{});
        }
      }
    }
  };

  // The ids of the window's rows, asked for together with its first expert: neither
  // waits for the other.
  if (tid < kMxRows) {
    const int r = window * win + tid;
    win_flat[tid] = (tid < win && r < win_end) ? p.sorted_ids[r] : -1;
  }
  int row = window * win;
  while (row < win_end) {  // uniform
    const int e = p.expert_ids[row / p.block_size];
    int seg_end = min(win_end, (row / p.block_size + 1) * p.block_size);
    while (seg_end < win_end && p.expert_ids[seg_end / p.block_size] == e)
      seg_end = min(win_end, seg_end + p.block_size);
    if (e >= 0) segment(row, seg_end - row, e);
    row = seg_end;
  }
}

template <int STAGE, int TERMS, bool PREACT = false>
bool mx_kernel_ready() {
  static const bool configured = [] {
    const hipError_t err = hipFuncSetAttribute(
        reinterpret_cast<const void*>(tile_mx_kernel<STAGE, TERMS, PREACT>),
        hipFuncAttributeMaxDynamicSharedMemorySize, kMxRing * kMxRows * TERMS * 128);
    if (err != hipSuccess) (void)hipGetLastError();  // not left for the next caller to find
    return err == hipSuccess;
  }();
  return configured;
}

template <int STAGE, int TERMS, bool PREACT = false>
void launch_mx_stage_t(MxArgs g, hipStream_t stream) {
  const int win = mx_window_rows(g.block_size);
  g.units = mx_units(STAGE, g.ncols);
  g.col_groups = (g.units + kMxWaves - 1) / kMxWaves;
  g.windows = (g.num_blocks * g.block_size + win - 1) / win;
  const long long total = (long long)g.col_groups * g.windows;
  const unsigned grid = (unsigned)((total + 255) / 256 * 256);  // whole chunks of 32 tiles for each of 8 XCDs
  hipLaunchKernelGGL((tile_mx_kernel<STAGE, TERMS, PREACT>), dim3(grid), dim3(64 * kMxWaves),
                     kMxRing * kMxRows * TERMS * 128, stream, g);
}

MxArgs mx_args(const FusedMoeArgs& a, int stage) {
  MxArgs g{};
  g.sorted_ids = a.sorted_ids;
  g.expert_ids = a.expert_ids;
  g.topk_w = a.topk_w;
  g.act = a.act;
  g.n_flat = a.M * a.top_k;
  g.top_k = a.top_k;
  g.num_blocks = a.EM / a.block_size;
  g.block_size = a.block_size;
  g.swiglu_limit = a.swiglu_limit;
  g.beta = a.beta;
  g.linear_beta = a.linear_beta;
  g.activation = a.activation;
  if (stage == 0) {
    g.A = a.A; g.bias = a.b13; g.K = a.hidden; g.ncols = a.ispp;
  } else {
    g.A = a.act; g.bias = a.b2; g.K = a.ispp; g.ncols = a.hidden;
  }
  g.a_stride = g.K;
  return g;
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

// ---- prepacked weights -------------------------------------------------------

size_t moe_prepack_bytes(int num_experts, int rows, int K, int stage) {
  if (num_experts <= 0 || rows <= 0 || K <= 0) return 0;
  const int ncols = stage == 0 ? rows / 2 : rows;
  const size_t units = (size_t)mx_units(stage, ncols);
  return mx_packed_bytes(num_experts, units, mx_kp(K) / 128);
}

void launch_moe_prepack(const uint8_t* w, const uint8_t* w_scale, int num_experts, int rows, int K,
                        int stage, uint8_t* packed, hipStream_t stream) {
  const int ncols = stage == 0 ? rows / 2 : rows;
  const int units = mx_units(stage, ncols);
  const int ksteps = mx_kp(K) / 128;
  uint8_t* flags = packed + mx_packed_body_bytes(num_experts, units, ksteps);
  hipLaunchKernelGGL(prepack_flag_kernel, dim3(units, num_experts), dim3(256), 0, stream, w, w_scale,
                     flags, stage, rows, ncols, K, units);
  hipLaunchKernelGGL(prepack_kernel, dim3(ksteps, units, num_experts), dim3(256), 0, stream, w,
                     w_scale, packed, flags, stage, rows, ncols, K, units, ksteps);
}

// ---- workspace of the prepacked path -------------------------------------------
//   split rows of A [M, 3 Kp(hidden)], of act [EM, 3 Kp(ispp)], their row flags,
//   the second stage's rows y [EM, hidden] fp32, pos [M top_k].

namespace {
struct MxWorkspace {
  size_t aq, cq, abad, cbad, y, pos;
  size_t total() const { return aq + cq + abad + cbad + y + pos; }
};
MxWorkspace mx_workspace(int M, int hidden, int ispp, int top_k, int EM) {
  MxWorkspace l;
  l.aq = align256((size_t)M * 3 * mx_kp(hidden));
  l.cq = align256((size_t)EM * 3 * mx_kp(ispp));
  l.abad = align256((size_t)M);
  l.cbad = align256((size_t)EM);
  l.y = align256((size_t)EM * hidden * sizeof(float));
  l.pos = align256((size_t)M * top_k * sizeof(int32_t));
  return l;
}
}  // namespace

size_t mx_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM) {
  return mx_workspace(M, hidden, ispp, top_k, EM).total();
}

bool prepare_mx_kernels() {
  return mx_kernel_ready<0, 1>() && mx_kernel_ready<0, 2>() && mx_kernel_ready<0, 3>() &&
         mx_kernel_ready<1, 1>() && mx_kernel_ready<1, 2>() && mx_kernel_ready<1, 3>() &&
         mx_kernel_ready<0, 2, true>() && mx_kernel_ready<0, 3, true>() && mx_kernel_ready<1, 2, true>() &&
         mx_kernel_ready<1, 3, true>();
}

namespace {

constexpr int kMxShortK = 1024;  // second-stage sums shorter than this take three terms by default

struct MxPlan {
  MxArgs g0, g1;
  uint8_t *aq, *cq, *abad, *cbad;
  float* y;
  int32_t* pos;
  // FP6 terms per activation in the first and in the second stage (2 or 3), or 1 and 1 =
  // the W4A4 mode (MXFP4 activations)
  int terms0, terms1;
};

// False when the prepacked path does not take the call (no packed weights, workspace
// short or misaligned, split rows beyond the 32-bit offsets of the row copies, LDS refused).
bool mx_plan(const FusedMoeArgs& a, bool need_stage0, MxPlan& pl) {
  if ((need_stage0 && a.w13_packed == nullptr) || a.w2_packed == nullptr || a.workspace == nullptr)
    return false;
  const MxWorkspace l = mx_workspace(a.M, a.hidden, a.ispp, a.top_k, a.EM);
  if (a.workspace_bytes < l.total() || (reinterpret_cast<uintptr_t>(a.workspace) & 15) != 0) return false;
  if ((unsigned long long)a.EM * 3ull * mx_kp(a.ispp) >= (1ull << 32) ||
      (unsigned long long)a.M * 3ull * mx_kp(a.hidden) >= (1ull << 32))
    return false;
  // VK_HIP_MOE_W4A4; _SPLIT2; _SPLIT3; default: three terms where the error passes through
  // the activation function and the second GEMM, two in the second stage -- but three
  // there as well when its sums are short (ispp < kMxShortK): the worst element's error
  // grows as the sums get shorter (1.7e-2 of the RMS at ispp = 64, 6.7e-3 at 256,
  // 4.6e-3 at 1024 and beyond with two terms; 2.5e-4 at 64 with three), and such
  // layers are small enough that the third term costs microseconds
  if ((a.flags & 4u) != 0u) pl.terms0 = pl.terms1 = 1;
  else if ((a.flags & 2u) != 0u) pl.terms0 = pl.terms1 = 2;
  else if ((a.flags & 8u) != 0u) pl.terms0 = pl.terms1 = 3;
  else { pl.terms0 = 3; pl.terms1 = a.ispp < kMxShortK ? 3 : 2; }
  const bool ready0 = !need_stage0 || (pl.terms0 == 1 ? mx_kernel_ready<0, 1>()
                                       : pl.terms0 == 2 ? mx_kernel_ready<0, 2>() : mx_kernel_ready<0, 3>());
  const bool ready1 = pl.terms1 == 1 ? mx_kernel_ready<1, 1>()
                      : pl.terms1 == 2 ? mx_kernel_ready<1, 2>() : mx_kernel_ready<1, 3>();
  if (!ready0 || !ready1) return false;
  uint8_t* base = static_cast<uint8_t*>(a.workspace);
  pl.aq = base;
  pl.cq = pl.aq + l.aq;
  pl.abad = pl.cq + l.cq;
  pl.cbad = pl.abad + l.abad;
  pl.y = reinterpret_cast<float*>(pl.cbad + l.cbad);
  pl.pos = reinterpret_cast<int32_t*>(pl.cbad + l.cbad + l.y);
  pl.g0 = mx_args(a, 0);
  pl.g1 = mx_args(a, 1);
  const int units0 = mx_units(0, a.ispp), units1 = mx_units(1, a.hidden);
  pl.g0.Wp = a.w13_packed;
  pl.g0.Wflags = a.w13_packed == nullptr ? nullptr :
      a.w13_packed + mx_packed_body_bytes(a.num_experts, units0, mx_kp(a.hidden) / 128);
  pl.g1.Wp = a.w2_packed;
  pl.g1.Wflags = a.w2_packed + mx_packed_body_bytes(a.num_experts, units1, mx_kp(a.ispp) / 128);
  pl.g0.Aq = pl.aq; pl.g0.row_bad = pl.abad;
  pl.g1.Aq = pl.cq; pl.g1.row_bad = pl.cbad;
  pl.g1.y = pl.y; pl.g1.pos = pl.pos;
  return true;
}

void mx_stage0(const FusedMoeArgs& a, const MxPlan& pl, hipStream_t stream) {
  if (pl.terms0 == 1) {
    hipLaunchKernelGGL(quant_rows_w4_kernel, dim3(a.M), dim3(256), 0, stream, a.A, pl.aq, pl.abad, a.hidden, nullptr, 0, nullptr, 0);
    launch_mx_stage_t<0, 1>(pl.g0, stream);
  } else if (pl.terms0 == 2) {
    hipLaunchKernelGGL(split_rows_fp6_kernel<2>, split_grid(a.M, a.hidden), dim3(256), 0, stream, a.A, pl.aq, pl.abad, a.hidden, a.hidden, a.M, nullptr, 0, nullptr, 0);
    launch_mx_stage_t<0, 2>(pl.g0, stream);
  } else {
    hipLaunchKernelGGL(split_rows_fp6_kernel<3>, split_grid(a.M, a.hidden), dim3(256), 0, stream, a.A, pl.aq, pl.abad, a.hidden, a.hidden, a.M, nullptr, 0, nullptr, 0);
    launch_mx_stage_t<0, 3>(pl.g0, stream);
  }
}

// split act (the routed rows of the sorted order; the same kernel clears the table of
// sorted positions) -> second stage -> per-token sum
void mx_stage1(const FusedMoeArgs& a, const MxPlan& pl, hipStream_t stream) {
  if (pl.terms1 == 1) {
    hipLaunchKernelGGL(quant_rows_w4_kernel, dim3(a.EM), dim3(256), 0, stream, a.act, pl.cq, pl.cbad, a.ispp, a.sorted_ids, a.M * a.top_k, pl.pos, a.M * a.top_k);
    launch_mx_stage_t<1, 1>(pl.g1, stream);
  } else if (pl.terms1 == 2) {
    hipLaunchKernelGGL(split_rows_fp6_kernel<2>, split_grid(a.EM, a.ispp), dim3(256), 0, stream, a.act, pl.cq, pl.cbad, a.ispp, a.ispp, a.EM, a.sorted_ids, a.M * a.top_k, pl.pos, a.M * a.top_k);
    launch_mx_stage_t<1, 2>(pl.g1, stream);
  } else {
    hipLaunchKernelGGL(split_rows_fp6_kernel<3>, split_grid(a.EM, a.ispp), dim3(256), 0, stream, a.act, pl.cq, pl.cbad, a.ispp, a.ispp, a.EM, a.sorted_ids, a.M * a.top_k, pl.pos, a.M * a.top_k);
    launch_mx_stage_t<1, 3>(pl.g1, stream);
  }
  launch_combine(pl.y, pl.pos, a.out, a.M, a.top_k, a.hidden, (a.flags & 1u) != 0u, stream);
}

}  // namespace

// The whole layer on prepacked weights; false when the path does not take the call
// (nothing has been enqueued then).
bool launch_fused_moe_prepacked(const FusedMoeArgs& a, hipStream_t stream) {
  MxPlan pl;
  if (!mx_plan(a, true, pl)) return false;
  mx_stage0(a, pl, stream);
  mx_stage1(a, pl, stream);
  return true;
}

// True when launch_fused_moe_prepacked (both_stages) or launch_moe_down_prepacked would
// take the call (nothing is enqueued).
bool fused_moe_prepacked_takes(const FusedMoeArgs& a, bool both_stages) {
  MxPlan pl;
  return mx_plan(a, both_stages, pl);
}

// The second stage alone (act is the caller's), likewise.
bool launch_moe_down_prepacked(const FusedMoeArgs& a, hipStream_t stream) {
  MxPlan pl;
  if (!mx_plan(a, false, pl)) return false;
  mx_stage1(a, pl, stream);
  return true;
}

// ---- the linear part of a stage on prepacked weights (tensor-parallel stage split) ----
// Workspace: split rows of the K slice [rows, 3 Kp(k_dim)] and a flag byte per row;
// rows = M (stage 0: the rows of A) or EM (stage 1: the sorted rows of act).
size_t mx_preact_workspace_bytes(int stage, int M, int EM, int k_dim) {
  if (M <= 0 || EM <= 0 || k_dim <= 0) return 0;
  const size_t rows = stage == 0 ? (size_t)M : (size_t)EM;
  return align256(rows * 3 * (size_t)mx_kp(k_dim)) + align256(rows);
}

// False (nothing enqueued) when the path does not take the call: workspace short or
// misaligned, split rows beyond 32-bit offsets, LDS refused.
bool launch_moe_preact_prepacked(int stage, const uint16_t* a, const uint8_t* packed, const uint8_t* w,
                                 const uint8_t* w_scale, const int32_t* sorted_ids, const int32_t* expert_ids,
                                 float* preact, int M, int a_stride, int ncols, int top_k, int EM, int k_base,
                                 int k_dim, int block_size, int num_experts, void* workspace,
                                 size_t workspace_bytes, unsigned flags, hipStream_t stream) {
  (void)w;  // (the exact path reads the packed form as well; the raw shard serves the
  (void)w_scale;  // small calls, which the caller runs on the raw-weight kernels)
  if (M <= 0 || EM <= 0 || block_size <= 0 || packed == nullptr || workspace == nullptr) return false;
  if (workspace_bytes < mx_preact_workspace_bytes(stage, M, EM, k_dim) ||
      (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
    return false;
  const size_t rows = stage == 0 ? (size_t)M : (size_t)EM;
  if ((unsigned long long)rows * 3ull * mx_kp(k_dim) >= (1ull << 32)) return false;
  // terms as in the layer: three in the first stage, two in the second unless its sums are
  // short; VK_HIP_MOE_SPLIT2 / _SPLIT3: that many
  int terms = stage == 0 ? 3 : (k_dim < kMxShortK ? 3 : 2);
  if ((flags & 2u) != 0u) terms = 2;
  else if ((flags & 8u) != 0u) terms = 3;
  const bool ready = stage == 0 ? (terms == 2 ? mx_kernel_ready<0, 2, true>() : mx_kernel_ready<0, 3, true>())
                                : (terms == 2 ? mx_kernel_ready<1, 2, true>() : mx_kernel_ready<1, 3, true>());
  if (!ready) return false;
  uint8_t* xq = static_cast<uint8_t*>(workspace);
  uint8_t* xbad = xq + align256(rows * 3 * (size_t)mx_kp(k_dim));
  MxArgs g{};
  g.sorted_ids = sorted_ids;
  g.expert_ids = expert_ids;
  g.n_flat = M * top_k;
  g.top_k = top_k;
  g.num_blocks = EM / block_size;
  g.block_size = block_size;
  g.A = a + k_base;
  g.a_stride = a_stride;
  g.K = k_dim;
  g.ncols = ncols;
  g.preact = preact;
  g.Aq = xq;
  g.row_bad = xbad;
  const int units = mx_units(stage, ncols);
  g.Wp = packed;
  g.Wflags = packed + mx_packed_body_bytes(num_experts, units, mx_kp(k_dim) / 128);
  const int32_t* ids = stage == 0 ? nullptr : sorted_ids;  // stage 1: the routed rows of the sorted order only
  const int n_flat = stage == 0 ? 0 : M * top_k;
  if (terms == 2)
    hipLaunchKernelGGL(split_rows_fp6_kernel<2>, split_grid((int)rows, k_dim), dim3(256), 0, stream, a + k_base, xq,
                       xbad, k_dim, a_stride, (int)rows, ids, n_flat, nullptr, 0);
  else
    hipLaunchKernelGGL(split_rows_fp6_kernel<3>, split_grid((int)rows, k_dim), dim3(256), 0, stream, a + k_base, xq,
                       xbad, k_dim, a_stride, (int)rows, ids, n_flat, nullptr, 0);
  if (stage == 0) {
    if (terms == 2) launch_mx_stage_t<0, 2, true>(g, stream);
    else launch_mx_stage_t<0, 3, true>(g, stream);
  } else {
    if (terms == 2) launch_mx_stage_t<1, 2, true>(g, stream);
    else launch_mx_stage_t<1, 3, true>(g, stream);
  }
  return true;
}

// Test hook: the split rows of bf16 rows [rows, K] as the GEMM kernels read them.
void launch_split_rows_fp6(const uint16_t* x, int rows, int K, int terms, uint8_t* xq, uint8_t* row_bad,
                           hipStream_t stream) {
  if (rows <= 0) return;
  if (terms == 2)
    hipLaunchKernelGGL(split_rows_fp6_kernel<2>, split_grid(rows, K), dim3(256), 0, stream, x, xq, row_bad, K, K, rows, nullptr, 0, nullptr, 0);
  else
    hipLaunchKernelGGL(split_rows_fp6_kernel<3>, split_grid(rows, K), dim3(256), 0, stream, x, xq, row_bad, K, K, rows, nullptr, 0, nullptr, 0);
}

// ---- MXFP4 orchestration ops (device counterparts of moe_aux.cpp) -----------------

void launch_mxfp4_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed, uint8_t* scales,
                        int rows, int hidden, int top_k, int n_flat, hipStream_t stream) {
  if (rows <= 0 || hidden <= 0) return;
  hipLaunchKernelGGL(mxfp4_quant_kernel, dim3(rows), dim3(256), 0, stream, A, sorted_ids, packed, scales,
                     hidden, top_k, n_flat);
}

}  // namespace vk
