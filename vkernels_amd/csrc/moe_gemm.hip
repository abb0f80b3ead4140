// moe_gemm.hip — the two grouped GEMMs of the fused MXFP4 MoE layer.
//
//   stage 0  act[r, 0:I]   = bf16(act_fn(A[tok(r)] . W13[e, 0:I]^T  + b13,
//                                        A[tok(r)] . W13[e, I:2I]^T + b13))
//   stage 1  out[tok(r), :] += (act[r] . W2[e]^T + b2) * topk_w[flat(r)]
//
// for every sorted row r of every block whose expert_ids entry e is >= 0
// (reference semantics: src/c/vkernels/kernels/moe_fused.cpp:235-564).
//
// Three kernels share the arithmetic (scaled FP4 x FP8 MFMA, see the decode
// kernel's comment) and the work decomposition:
//
//   * a run = the consecutive blocks of one expert (in the decode kernel every
//     block by itself); padding rows (sorted id >= M*top_k) and blocks with
//     expert id < 0 are skipped;
//   * a wavefront owns NT weight tiles of 16 rows each (stage 0: NT/2 gate
//     tiles and the NT/2 up tiles of the same columns, so the activation is
//     fused; stage 1: NT consecutive tiles) and walks the whole K dimension;
//   * weights sit on the A side of the MFMA: lane (n, q) = (lane % 16,
//     lane / 16) holds row n, so one global_load_dwordx4 of that lane brings
//     the 32 codes of one scale group -- the lane's whole operand for a K step
//     of 128; quad q takes group 4*step + q, so a wavefront reads 64
//     contiguous bytes of each of its 16 rows per step.  Weights never pass
//     through LDS;
//   * the activation rows are split into two E4M3 terms per block of 32 and
//     held in LDS as MFMA operands, shared by the workgroup's wavefronts;
//   * stage 1 adds into `out` with hardware fp32 atomics, as the ABI
//     requires `out` to be accumulated into.
//
// stream_resident_kernel: decode (few rows per expert, K up to 3072): HBM
//   bound, one workgroup per compute unit, all of K of 16 rows resident.  It has
//   a second form that reads the weights from the prepacked layout of
//   moe_prefill_layout.hpp instead (taken whenever the caller gives it: the
//   scale bytes then come with the codes and nothing is checked or moved in the
//   loop), and forms that align, or route and align, for themselves.
// tile_wide_kernel: everything else when the caller lends a workspace (and K >=
//   512): 128 rows x 16 weight tiles per workgroup, rows pre-split in the
//   workspace, operands brought to LDS by DMA three K steps ahead; the second
//   stage stores its rows and combine_kernel sums them per token.
// tile_gemm_kernel: everything else without a workspace: 64 rows x 16 weight
//   tiles per workgroup, K in chunks of 512, rows split in-kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <type_traits>

#include "moe_common.hpp"
#include "moe_heuristics.hpp"
#include "moe_prefill_layout.hpp"
#include "moe_route.hpp"
#include "moe_tuning.hpp"
#include "mxfp4.hpp"
#include "vk_internal.hpp"

namespace vk {
namespace {


struct GemmArgs {
  const uint16_t* A;        // stage 0: activations [M, K]; stage 1: act [EM, K]
  const uint8_t* W;         // [E, rows_w, K/2]
  const uint8_t* Ws;        // [E, rows_w, K/32]
  // The same weights in the prepacked form (moe_prefill_layout.hpp), for the decode
  // kernels' packed instantiations, which read nothing of W / Ws: the blocks, the flag
  // byte of every (expert, packed unit), packed units per expert.
  const uint8_t* Wp;
  const uint8_t* Wpf;
  int p_units;
  int p_experts;            // experts in the prepacked weights
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const float* topk_w;      // stage 1
  const float* bias;        // b13 [E, 2I] or b2 [E, H], may be null
  uint16_t* act;            // stage 0 output [EM, I]
  float* out;               // stage 1 output [M, H]
  // Optional "split rows" (workspace tile kernel): the bf16 rows of A already
  // split into the two E4M3 terms.  With Kp = split_row_k(K) (K rounded up to a
  // whole K step of 128), row r is 2 Kp bytes at Aq + r * 2 Kp: the leading parts
  // (K of them, then zeros up to Kp), then the remainders (times 16) likewise.
  // As[r * split_scale_stride(K) + g] is the scale byte of block g, 0 = block
  // outside the fast path's range, 127 for the blocks between K and Kp.
  const uint8_t* Aq;
  const uint8_t* As;
  uint8_t* actq;            // stage 0: act written in that form as well (or null)
  float* zero_out;          // stage 0: buffer to clear while the stage runs (or null)
  long long zero_count;     // its floats (a multiple of 4)
  uint8_t* actqs;
  // Stage 1, optional: instead of adding into `out`, row `srow` of the sorted rows goes
  // to y[srow, :] (bias and routing weight applied) and pos[flat] = srow; combine_kernel
  // then sums each token's rows.
  float* y;
  int32_t* pos;
  // Optional: the stage's linear part alone (tensor-parallel callers sum it over ranks
  // before the epilogue): stage 0 stores preact[srow, c] = gate and preact[srow, ncols + c]
  // = up of every routed sorted row (row width 2 ncols), stage 1 preact[srow, c] (width
  // ncols); no bias, no activation, no routing weight.
  float* preact;
  int a_stride;             // elements between rows of A (K, or the full width of a K slice)
  int n_flat;               // M * top_k
  int top_k;
  int K;                    // hidden (stage 0) or ispp (stage 1)
  int ncols;                // ispp (stage 0) or hidden (stage 1)
  int num_blocks;
  int block_size;
  float swiglu_limit, beta, linear_beta;
  int activation;
  // The routed form of the decode kernel's first stage (a handful of tokens): router and
  // alignment are done by every workgroup for itself, in LDS, from the logits; workgroup 0
  // writes the tables out for the second stage and the caller.  sorted_ids / expert_ids
  // above are not read then.
  const float* rt_logits;        // [M, rt_experts]
  const int32_t* rt_expert_map;  // or null
  int32_t* rt_topk_ids;          // [M, top_k] out
  float* rt_topk_w;              // [M, top_k] out
  int32_t* rt_sorted_ids;        // [rt_max_em] out
  int32_t* rt_expert_ids;        // [rt_max_em / 16] out
  int32_t* rt_out_em;            // out
  int rt_experts, rt_local_n, rt_renormalize, rt_max_em;
};

// Rows a tile-kernel workgroup takes at a time: the largest multiple of 16 that
// divides the block size and does not exceed `max_rows` (a group never spans
// two blocks, hence never two experts).
__host__ __device__ inline int tile_group_rows(int block_size, int max_rows) {
  for (int rows = max_rows; rows > 16; rows -= 16)
    if (block_size % rows == 0) return rows;
  return 16;
}

// Bytes between the scale rows of split rows: K/32 rounded up to 16.
__host__ __device__ inline int split_scale_stride(int K) { return (K / 32 + 15) & ~15; }

// Values per term of a split row: K rounded up to a whole K step.
__host__ __device__ inline int split_row_k(int K) { return (K + 127) & ~127; }

// Stage 0 of a call that was asked to overwrite `out`: every workgroup clears
// its share (the stage does not use `out`; the next stage starts after this one).
// THREADS = the workgroup's size, known to every caller at compile time.
template <int THREADS>
__device__ __forceinline__ void clear_out_share(const GemmArgs& p) {
  if (p.zero_out == nullptr) return;
  const long long n4 = p.zero_count / 4;
  const long long wg = (long long)blockIdx.y * gridDim.x + blockIdx.x;
  const long long wgs = (long long)gridDim.x * gridDim.y;
  f32x4* out4 = reinterpret_cast<f32x4*>(p.zero_out);
  for (long long i = wg * THREADS + threadIdx.x; i < n4; i += wgs * THREADS)
    out4[i] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// Epilogue of one 16-row activation tile: acc[t][r] = C[weight row 4*lq + r of
// tile t][activation row ln].  Stage 0 applies bias + activation to the
// (gate, up) pairs and stores bf16; stage 1 applies bias and the routing
// weight and adds into `out`.
// Stage 0 also returns what it stored: packed[t] = the 4 bf16 act values of tile pair t.
template <int STAGE, int NT>
__device__ __forceinline__ void epilogue_tile(const GemmArgs& p, int e, const f32x4 (&acc)[NT],
                                              const int (&col0)[NT], int flat, int srow, int lq,
                                              uint2* packed_out = nullptr) {
  if (p.preact != nullptr) {  // the linear part alone, as fp32
    const int width = STAGE == 0 ? 2 * p.ncols : p.ncols;
    float* row = p.preact + (size_t)srow * (size_t)width;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int c = col0[t] + 4 * lq + ((STAGE == 0 && t >= NT / 2) ? p.ncols : 0);
      *reinterpret_cast<f32x4*>(row + c) = acc[t];
    }
    return;
  }
  if (STAGE == 0) {
#pragma unroll
    for (int t = 0; t < NT / 2; ++t) {
      const int c = col0[t] + 4 * lq;
      f32x4 gate = acc[t], up = acc[t + NT / 2];
      if (p.bias != nullptr) {  // uniform; the lane's four columns in one load each
        const float* b = p.bias + (size_t)e * (size_t)(2 * p.ncols) + c;
        gate += *reinterpret_cast<const f32x4u*>(b);
        up += *reinterpret_cast<const f32x4u*>(b + p.ncols);
      }
      uint32_t packed[2];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = gate[r];
        const float u = up[r];
        const uint32_t v = f32_to_bf16_bits(
            act_value(p.activation, g, u, p.swiglu_limit, p.beta, p.linear_beta));
        if (r & 1) packed[r >> 1] |= v << 16;
        else packed[r >> 1] = v;
      }
      *reinterpret_cast<uint2*>(p.act + (size_t)srow * (size_t)p.ncols + c) =
          make_uint2(packed[0], packed[1]);
      if (packed_out != nullptr) packed_out[t] = make_uint2(packed[0], packed[1]);
    }
  } else {
    const float w = p.topk_w[flat];
    float* orow = p.out + (size_t)(flat / p.top_k) * (size_t)p.ncols;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int c = col0[t] + 4 * lq;
      f32x4 v = acc[t];
      if (p.bias != nullptr)  // uniform
        v += *reinterpret_cast<const f32x4u*>(p.bias + (size_t)e * (size_t)p.ncols + c);
#pragma unroll
      for (int r = 0; r < 4; ++r) unsafeAtomicAdd(orow + c + r, v[r] * w);
    }
  }
}

// Second stage of the decode kernels: the same tile the other way round,
// acc[t][r] = C[activation row 4*lq + r][weight row ln of tile t] (the kernels give the
// matrix cores the rows as the first operand there).  The 16 lanes of a quarter then add
// into 16 consecutive floats of one row of `out`, a whole 64-byte sector an instruction,
// where the layout above has four lanes to a sector and sixteen sectors an instruction:
// the atomic units take a request per sector, and a step's additions cost a tenth.
// flat4[r] = the flat index of row 4*lq + r of the tile (< 0: padding), w4[r] its routing
// weight (rows_weights below: asked for when the rows are listed, not here, where a load
// would have every weight load in flight waited for first), srow0 = the tile's first
// sorted row.
__device__ __forceinline__ void rows_weights(const GemmArgs& p, const int (&flat4)[4], float (&w4)[4]) {
  if (p.topk_w == nullptr) {  // (the linear part alone)
#pragma unroll
    for (int r = 0; r < 4; ++r) w4[r] = 0.f;
    return;
  }
  // no load under a condition: one that is skipped by its lanes would still be waited for
#pragma unroll
  for (int r = 0; r < 4; ++r) w4[r] = p.topk_w[max(flat4[r], 0)];
}

template <int NT>
__device__ __forceinline__ void epilogue_rows(const GemmArgs& p, int e, const f32x4 (&acc)[NT],
                                              const int (&col0)[NT], const int (&flat4)[4],
                                              const float (&w4)[4], int srow0, int lane) {
  const int ln = lane & 15, lq = lane >> 4;
  if (p.preact != nullptr) {  // the linear part alone, as fp32
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (flat4[r] < 0) continue;
      float* row = p.preact + (size_t)(srow0 + 4 * lq + r) * (size_t)p.ncols;
#pragma unroll
      for (int t = 0; t < NT; ++t) row[col0[t] + ln] = acc[t][r];
    }
    return;
  }
  float b[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) b[t] = 0.f;
  if (p.bias != nullptr) {  // uniform
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      b[t] = p.bias[(size_t)e * (size_t)p.ncols + col0[t] + ln];
      __asm__ volatile("" : "+v"(b[t]));  // (waited for here, by every lane)
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (flat4[r] < 0) continue;
    float* orow = p.out + (size_t)(flat4[r] / p.top_k) * (size_t)p.ncols + ln;
#pragma unroll
    for (int t = 0; t < NT; ++t) unsafeAtomicAdd(orow + col0[t], (acc[t][r] + b[t]) * w4[r]);
  }
}

// Weight rows, scale rows and first output column of the NT tiles of `unit`.
template <int STAGE, int NT>
__device__ __forceinline__ void unit_tiles(const GemmArgs& p, int e, int unit, int ln,
                                           const uint8_t* (&w_rows)[NT],
                                           const uint8_t* (&s_rows)[NT], int (&col0)[NT]) {
  const int rows_w = STAGE == 0 ? 2 * p.ncols : p.ncols;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int row;
    if (STAGE == 0) {
      const int half = t / (NT / 2), tt = t % (NT / 2);
      col0[t] = unit * (8 * NT) + tt * 16;
      row = half * p.ncols + col0[t] + ln;
    } else {
      col0[t] = unit * (16 * NT) + t * 16;
      row = col0[t] + ln;
    }
    const size_t r = (size_t)e * (size_t)rows_w + (size_t)row;
    w_rows[t] = p.W + r * (size_t)(p.K / 2);
    s_rows[t] = p.Ws + r * (size_t)(p.K / 32);
  }
}

// The same for the prepacked form.  A decode tile (16 weight rows from row c of the gate,
// up or down matrix, c a multiple of 16) lies inside one 32-row tile of one packed unit:
// unit c / 64 (gate / up: tiles 0, 1 / 2, 3 of it) or c / 128 (down), rows c % 32 .. + 15
// of tile (c % 64) / 32 resp. (c % 128) / 32.  Lane (ln, lq) takes K block lq of row ln of
// the step: half lq / 2, lane (lq % 2, c % 32 + ln) of the packed tile.  w_rows / s_rows
// point at that lane's 16 code bytes and at the four scale bytes of its half (the tile's
// is byte shift / 8 of them) in the unit's first K step; every further step is
// kMxStepBytes on.  pu = the packed unit (the same for all tiles of a decode unit).
template <int STAGE, int NT>
__device__ __forceinline__ void unit_tiles_packed(const GemmArgs& p, int e, int unit, int lane, int nsteps,
                                                  const uint8_t* (&w_rows)[NT],
                                                  const uint8_t* (&s_rows)[NT], int (&shift)[NT],
                                                  int (&col0)[NT], int& pu) {
  static_assert(NT <= 2, "a decode unit lies inside one packed unit");
  const int ln = lane & 15, lq = lane >> 4;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int c, ptile;
    if (STAGE == 0) {
      const int half = t / (NT / 2), tt = t % (NT / 2);
      col0[t] = unit * (8 * NT) + tt * 16;
      c = col0[t];
      pu = c >> 6;
      ptile = half * 2 + ((c & 63) >> 5);
    } else {
      col0[t] = unit * (16 * NT) + t * 16;
      c = col0[t];
      pu = c >> 7;
      ptile = (c & 127) >> 5;
    }
    const int ln32 = (c & 31) + ln;
    const uint8_t* ub = p.Wp + mx_unit_offset(e, p.p_units, pu, nsteps);
    w_rows[t] = ub + (lq >> 1) * 4096 + ptile * 1024 + (lq & 1) * 512 + ln32 * 16;
    s_rows[t] = ub + 8192 + ((lq & 1) * 32 + ln32) * 8 + (lq >> 1) * 4;
    shift[t] = 8 * ptile;
  }
}

// Flag byte of a packed unit (non-zero = it holds a code or a scale byte the fast path does
// not take, and its codes and scale bytes are the raw tensors').  The index is uniform, so
// the word that holds the byte comes through the scalar path (a read of memory that no
// kernel writes while this one runs; the flags start on a multiple of 256 bytes and are
// padded to one): it does not queue with the vector loads, and a wait for it waits for
// nothing else.  The caller keeps the word and looks at it when the unit is complete.
__device__ __forceinline__ uint32_t packed_unit_flag(const GemmArgs& p, int e, int pu) {
  typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;
  const int idx = __builtin_amdgcn_readfirstlane(e * p.p_units + pu);
  const uintptr_t word = reinterpret_cast<uintptr_t>(p.Wpf) + (uintptr_t)(idx & ~3);
  return (*(const_u32_ptr)word >> (8 * (idx & 3))) & 0xFFu;
}

// ---------------------------------------------------------------------------
// Decode kernel ("resident"): one workgroup per compute unit, the activation
// rows of a run resident in LDS for the whole K dimension, no barrier inside
// the K loop, every wavefront's weight loads one uninterrupted stream, and
// the FP4 codes fed to the matrix cores as they are.
//
// Arithmetic.  v_mfma_scale_f32_16x16x128_f8f6f4 multiplies an FP4 (E2M1)
// operand by an FP8 (E4M3) operand, each with one E8M0 scale per lane that
// covers the lane's block of 32 along K.  The weight side is the packed codes
// moved onto the OCP code points (mxfp4.hpp: +2 on codes with a non-zero
// exponent field, scale byte - 1), 16 bytes = one scale group = one lane.
// The bf16 activations are split, per block of 32, as
//     a = (hi + lo / 16) * 2^(sb - 127),   hi, lo in E4M3,
// with sb = (largest exponent field of the block) - 7: hi takes the leading
// four significant bits of a / 2^(sb-127), lo the other four, so the split is
// exact for every element within 2^-13 of the block's largest and the two
// MFMAs (hi, then lo with scale byte sb - 4) sum the same products the
// reference forms, in fp32.
// A unit whose weights hold an inf/NaN code or a scale byte outside
// [kScaleLo, kScaleHi], and a pass whose activations hold an inf/NaN or a
// block exponent outside that range, are computed by exact_unit_global
// instead: integer-exact dequantisation, bf16 MFMAs, activations from global
// memory.
//
// Work split.  The launch has as many workgroups as the device has compute
// units.  Every workgroup lists the runs (every block with an expert by
// itself, so that with blocks of 16 rows the 16-row passes over an expert's
// weights run side by side in different workgroups, each staging its rows
// once), flattens (run, weight unit) into one index space and takes a contiguous
// slice of it (kStagingUnits below), so the weight bytes are spread evenly over
// the compute units whatever the number of active experts.  For each run its
// slice touches, and each 16-row pass of that run, the workgroup stages the
// 16 activation rows, all of K, into LDS as MFMA operands (split as above).
// Wavefront w takes units w, w + WAVES, ... of the slice and walks their K
// steps as ONE sequence: a D-deep register pipeline of 16-byte-per-lane
// weight loads whose cursor runs ahead of the arithmetic and crosses from one
// unit into the next.  The scale bytes of a unit (16 rows x K/32, contiguous
// per tile) are fetched with a few coalesced loads while the previous unit
// streams and parked in a per-wavefront LDS region.
//
// Start-up.  Until the stream runs, a workgroup is a chain of dependent steps
// on an otherwise idle compute unit, where every instruction and every round
// trip to memory is paid in full (about 10 us of a 65 us kernel at 2880 x
// 2880 x 32 experts, 64 tokens).  So: wavefront 0 lists the runs with one
// round trip (a block's expert and both neighbours' loaded together) and
// finds the slice with ballots, a lane per run, no reductions; meanwhile the
// other wavefronts copy the head of sorted_ids to LDS, so the ids of the first
// rows are an LDS read; offsets that depend on the piece index alone are
// compile-time constants (a wavefront's pieces keep their quarter of a K
// step); the scale pieces of a unit are addressed without divisions.
//
// Order within a pass.  The memory pipe of a compute unit returns data in the
// order of issue, and the stream cannot start before the rows are staged, so:
// (1) the row ids, (2) the rows, (3) the first D steps of the weight stream,
// which then are on their way while the rows are checked, split and written,
// then the barrier with the previous pass.  The rows are split and written in
// K order, a few K steps ahead of the first unit's arithmetic with a barrier
// after each portion, so the stream starts after the first portion and the
// rest of the splitting overlaps it.
//
// LDS operand planes of K step ks: [term hi/lo][half h][64 lanes] x 16 bytes;
// lane (n, q') of half h holds the 16 values k = 128 ks + 64 h + 16 q' + 0..15
// of row n, which is where the MFMA takes them from (operand bytes 16 h ..
// 16 h + 15).  Planes past K are zero, so the last, partial K step needs no
// masking of the weight side.
// ---------------------------------------------------------------------------
constexpr int kMaxRuns = kMoeMaxRuns;   // runs the resident kernel can list in LDS
// 16-byte scale pieces of a unit a lane holds: NT * K/32 <= 64 * resident_scale_pieces.
// Workgroups of 8 wavefronts stage K <= 3072 (resident_batch), 96 groups, and have
// 256 registers a lane: three pieces are enough there, and a fourth would cost four registers.
__host__ __device__ constexpr int resident_scale_pieces(int waves) { return waves == 4 ? 4 : 3; }

typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;

// Two 16-byte LDS reads as the 32-byte FP8 operand of the scaled MFMA.
__device__ __forceinline__ i32x8 fp8_operand(u32x4 lo16, u32x4 hi16) {
  typedef __attribute__((ext_vector_type(8))) uint32_t u32x8;
  const u32x8 v = __builtin_shufflevector(lo16, hi16, 0, 1, 2, 3, 4, 5, 6, 7);
  return (i32x8)v;
}

// The 32 codes of one lane as the FP4 operand of the scaled MFMA: moved onto the
// OCP code points, in the low four of the operand's eight registers (the
// instruction does not read the other four for FP4, so they are left undefined).
__device__ __forceinline__ i32x8 fp4_operand(u32x4 w) {
  const i32x4 y = {(int)fp4x8_to_ocp_doubled(w[0]), (int)fp4x8_to_ocp_doubled(w[1]),
                   (int)fp4x8_to_ocp_doubled(w[2]), (int)fp4x8_to_ocp_doubled(w[3])};
  return __builtin_shufflevector(y, y, 0, 1, 2, 3, -1, -1, -1, -1);
}

// The same for codes that are on the OCP code points already (the prepacked form).
__device__ __forceinline__ i32x8 fp4_operand_packed(u32x4 w) {
  const i32x4 y = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  return __builtin_shufflevector(y, y, 0, 1, 2, 3, -1, -1, -1, -1);
}

// Position of a workgroup in the decode kernels' split of the work.  The hardware hands
// consecutive workgroup ids to the 8 XCDs in turn, each with an L2 of its own.  Taking the
// ids of one XCD as one consecutive range of positions puts the workgroups of a run, and of
// the runs next to it, behind one L2: the passes of an expert with several blocks are runs
// side by side whose workgroups stream the same weights at the same time, so what the first
// of them fetches the others find there.
__device__ __forceinline__ int xcd_major_index(int id, int grid) {
  return (grid & 7) == 0 ? (id & 7) * (grid >> 3) + (id >> 3) : id;
}

// First item of part `i` when `total` items are cut into `parts` contiguous
// slices whose sizes differ by at most one.
__device__ __forceinline__ int slice_begin(int total, int i, int parts) {
  const int q = total / parts, rem = total - q * parts;
  return i * q + min(i, rem);
}

// A workgroup's slice [s0, s1) of the flat (run, unit) space.
//
// Streaming a run's units costs (units) x (its 16-row passes), and staging the
// rows of a run costs about as much as streaming kStagingUnits units.  So when
// every run can have workgroups of its own, run r gets a share of the grid
// proportional to its passes (taken as its 16-row tiles, an upper bound that
// is exact for block size 16) and the slices stop at run boundaries, provided
// that gives every run a workgroup and does not unbalance the workgroups by
// more than a second staging would cost.  Otherwise the space is cut evenly
// and a slice may span runs.
constexpr int kStagingUnits = 4;

// Reference-exact slow path for one unit: one K step at a time, integer-exact
// dequantisation, the activation row of this lane's column read from global
// memory (a_row null = padding row).
// ROWS_FIRST: the activation rows as the first operand (the tile the other way round, for
// epilogue_rows).
template <int NT, bool ROWS_FIRST = false>
__device__ __forceinline__ void exact_unit_global(const uint8_t* const (&w_rows)[NT],
                                                  const uint8_t* const (&s_rows)[NT],
                                                  const uint16_t* a_row, int K, int lane,
                                                  f32x4 (&acc)[NT]) {
  const int lq = lane >> 4;
  const int groups = K / 32;
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int ks = 0; ks * 4 < groups; ++ks) {
    const int g = ks * 4 + lq;
    const bool ok = g < groups;
#pragma unroll 1
    for (int d = 0; d < 4; ++d) {
      u32x4 av = {0u, 0u, 0u, 0u};
      if (ok && a_row != nullptr) av = *reinterpret_cast<const u32x4*>(a_row + g * 32 + d * 8);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        uint32_t x = 0u, sc = 127u;
        if (ok) {
          x = *reinterpret_cast<const uint32_t*>(w_rows[t] + (size_t)g * 16 + d * 4);
          sc = s_rows[t][g];
        }
        if constexpr (ROWS_FIRST)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av), as_bf16x8(dequant8_exact(x, sc)),
                                                           acc[t], 0, 0, 0);
        else
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(dequant8_exact(x, sc)),
                                                           as_bf16x8(av), acc[t], 0, 0, 0);
      }
    }
  }
}

// The same from the prepacked form (pointers of unit_tiles_packed).  raw: the unit is
// flagged and holds the raw codes and scale bytes; otherwise the move onto the OCP code
// points and the decrement of the scale byte are undone (all codes of such a unit are finite).
template <int NT, bool ROWS_FIRST = false>
__device__ __forceinline__ void exact_unit_packed(const uint8_t* const (&w_rows)[NT],
                                                  const uint8_t* const (&s_rows)[NT],
                                                  const int (&shift)[NT], bool raw, const uint16_t* a_row,
                                                  int K, int lane, f32x4 (&acc)[NT]) {
  const int lq = lane >> 4;
  const int groups = K / 32;
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int ks = 0; ks * 4 < groups; ++ks) {
    const int g = ks * 4 + lq;
    const bool ok = g < groups;
#pragma unroll 1
    for (int d = 0; d < 4; ++d) {
      u32x4 av = {0u, 0u, 0u, 0u};
      if (ok && a_row != nullptr) av = *reinterpret_cast<const u32x4*>(a_row + g * 32 + d * 8);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        uint32_t x = 0u, sc = 127u;
        if (ok) {
          x = *reinterpret_cast<const uint32_t*>(w_rows[t] + (size_t)ks * kMxStepBytes + d * 4);
          sc = (*reinterpret_cast<const uint32_t*>(s_rows[t] + (size_t)ks * kMxStepBytes) >> shift[t]) & 0xFFu;
          if (!raw) {
            x -= (x & 0x44444444u) >> 1;
            sc = (sc + 1u) & 0xFFu;
          }
        }
        if constexpr (ROWS_FIRST)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av), as_bf16x8(dequant8_exact(x, sc)),
                                                           acc[t], 0, 0, 0);
        else
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(dequant8_exact(x, sc)),
                                                           as_bf16x8(av), acc[t], 0, 0, 0);
      }
    }
  }
}

// 8 bf16 values -> the 8 E4M3 leading parts of v / 2^(sb-127) and the 8 E4M3
// remainders times 16.  gfx950's scaled conversions divide by the scale on the
// way down to FP8 and multiply by it on the way up.
__device__ __forceinline__ void split_bf16x8(u32x4 v, uint32_t sb, uint2& hi, uint2& lo) {
  typedef __attribute__((ext_vector_type(2))) short i16x2;
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  const float scale = __uint_as_float(sb << 23);
  const float scale16 = __uint_as_float((sb - 4u) << 23);
  union Pack { i16x2 h; uint32_t u; };
  Pack h[2], l[2];
  h[0].u = h[1].u = l[0].u = l[1].u = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    union { uint32_t u; bf16x2 b; } x;
    x.u = v[i];
    if (i & 1) h[i >> 1].h = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(h[i >> 1].h, x.b, scale, true);
    else h[i >> 1].h = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(h[i >> 1].h, x.b, scale, false);
    f32x2 back;
    if (i & 1) back = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(h[i >> 1].u, scale, true);
    else back = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(h[i >> 1].u, scale, false);
    const float r0 = __uint_as_float(v[i] << 16) - back[0];
    const float r1 = __uint_as_float(v[i] & 0xFFFF0000u) - back[1];
    if (i & 1) l[i >> 1].h = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(l[i >> 1].h, r0, r1, scale16, true);
    else l[i >> 1].h = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(l[i >> 1].h, r0, r1, scale16, false);
  }
  hi = make_uint2(h[0].u, h[1].u);
  lo = make_uint2(l[0].u, l[1].u);
}

// 16-byte pieces of a row that a lane of the resident kernel holds in registers while it
// stages a pass (every wavefront takes every WAVES-th group of 32 values): workgroups of
// 8 wavefronts, two to a SIMD, hold K <= 3072; workgroups of 4, with a SIMD's whole
// register file each, K <= 4096.
// (wide: the WIDEK instantiations on the prepacked weights, which have the registers for
// K <= 4096 with 8 wavefronts as well: no scale block to hold.)
__host__ __device__ constexpr int resident_batch(int waves, bool wide = false) {
  return waves == 4 ? 32 : (wide ? 128 : 96) / waves;
}

// KSPLIT: the form for a handful of rows (one token), where a workgroup's slice is fewer
// units than half its wavefronts and a unit, a chain of K / 128 dependent steps with D in
// flight, is all a wavefront would do while most have nothing.  The slice is taken at most
// WAVES / 2 units at a time; the WAVES / units wavefronts of a unit take a part of its K
// steps each, all rows are staged before any of them starts, and the unit's first wavefront
// adds the others' sums (through LDS, over the operand planes, in a fixed order) and runs
// the epilogue, or the exact path if any part met a value outside the fast path's domain.
// ROUTE (first stage, blocks of 16 rows, at most kRouteMaxRows routed rows): the router and
// the alignment run inside the kernel, so that a decode step of a handful of tokens is two
// launches and not three.  Every workgroup routes all the tokens itself (a wavefront per
// token, the arithmetic of route_topk_kernel), counts the rows of every local expert,
// gives every expert with rows its blocks in ascending order -- these are the runs -- and
// ranks every routed row inside its expert's blocks, all in LDS, which is what
// route_align_kernel does per workgroup as well; workgroup 0 also writes topk_ids, topk_w,
// sorted_ids, expert_ids and EM out, exactly as vk_hip_moe_route_align leaves them.
// ROUTE = 2 is the same without the router: topk_ids comes from the router's own launch
// (with more than a handful of tokens every workgroup routing all of them costs more than
// that launch) and the kernel only aligns, which saves the alignment's launch and this
// kernel's listing of the runs.
constexpr int kRouteMaxRows = kMoeRoutedMaxRows, kRouteMaxExperts = 256, kRoutePer = kRouteMaxExperts / 64;
constexpr int kRouteMaxTokens = 16;  // ROUTE = 1: tokens every workgroup routes for itself

// A workgroup barrier for LDS alone.  __syncthreads() is a workgroup-wide fence as well,
// which makes a wavefront wait for every global load it has in flight (s_waitcnt vmcnt(0)):
// in the decode kernel that is the weight stream and the rest of the rows, asked for on
// purpose before the barrier.  Only LDS is shared across these barriers; registers that
// global loads fill are waited for where they are used.
__device__ __forceinline__ void lds_barrier() {
  __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// PACKED: the weights are read from the prepacked form (GemmArgs::Wp) and W / Ws not at
// all, so that a caller who prepacks needs no second copy of the weights.  A lane's 16
// code bytes of a K step are where unit_tiles_packed says, already on the OCP code points,
// and the scale bytes (already less one) come with the step, four to a lane, so there is
// no scale block to park in LDS and nothing to check in the loop: a unit that needs the
// exact path carries a flag, looked up when the unit is begun.
// WIDEK: rows of 3072 < K <= 4096 with 8 wavefronts (16 row pieces a lane instead of 12): the
// prepacked form has the registers for it; an instantiation of its own, because the four
// more pieces cost the narrower rows a microsecond a kernel.
template <int STAGE, int WAVES, int NT, int D, bool KSPLIT = false, int ROUTE = 0, bool PACKED = false,
          bool WIDEK = false>
__global__ __launch_bounds__(64 * WAVES) void stream_resident_kernel(GemmArgs p) {
  static_assert(!WIDEK || (PACKED && WAVES == 8 && STAGE == 0), "the wide rows are the first stage's, prepacked form");
  static_assert(ROUTE == 0 || STAGE == 0, "the routed form is the first stage's");
  static_assert(ROUTE == 0 || 64 * WAVES >= kRouteMaxRows, "a lane per routed row");
  static_assert(!PACKED || (WAVES * (STAGE == 0 ? 8 * NT : 16 * NT)) % (STAGE == 0 ? 64 : 128) == 0,
                "a wavefront's consecutive units are whole packed units apart");
  extern __shared__ u32x4 b_lds[];  // [nsteps][2][2][64] operand planes, block scales, weight scales
  __shared__ int run_block0[kMaxRuns];
  __shared__ int run_expert[kMaxRuns];
  __shared__ int run_cum[kMaxRuns];     // blocks of the runs up to and including this one
  // routed form: local expert of every routed row, rows per local expert (then the first
  // block of the expert), the 16 flat indices of every run (0xFF = padding), the run count
  __shared__ short rt_le[ROUTE ? kRouteMaxRows : 1];
  __shared__ int rt_hist[ROUTE ? kRouteMaxExperts : 1];
  __shared__ unsigned short run_ids[ROUTE ? kRouteMaxRows * 16 : 1];
  // ... rows of every local expert among the 64 routed rows a wavefront ranks
  __shared__ int rt_cnt[ROUTE ? kRouteMaxRows / 64 : 1][ROUTE ? kRouteMaxExperts : 1];
  __shared__ int rt_runs;
  __shared__ int slice_sh[2];           // this workgroup's slice of the (run, unit) space
  __shared__ int pass_slow[2];          // set while staging: this pass takes the exact path
  __shared__ int ks_bad[KSPLIT ? WAVES : 1];  // K split: a wavefront's part of its unit left the fast path
  if (STAGE == 0) clear_out_share<64 * WAVES>(p);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and known to be
  const int ln = lane & 15;
  const int lq = lane >> 4;

  const int K = p.K;
  const int groups = K / 32;
  const int nsteps = (groups + 3) / 4;  // K steps, the last one possibly partial
  const int units = STAGE == 0 ? p.ncols / (8 * NT) : p.ncols / (16 * NT);
  const int sc_tile_bytes = 16 * groups;  // scale bytes of one 16-row tile
  uint8_t* bsc_lds = reinterpret_cast<uint8_t*>(b_lds + (size_t)nsteps * 256);  // [nsteps][64]
  uint8_t* sc_lds = bsc_lds + (size_t)nsteps * 64 + (size_t)wave * NT * sc_tile_bytes;  // (not PACKED)
  // rows of W between the units a wavefront takes one after the other
  const size_t unit_stride_rows = (size_t)WAVES * (STAGE == 0 ? 8 * NT : 16 * NT);
  // packed units between them, and the bytes: of W (PACKED: of the packed form) and of Ws
  constexpr int kPackedStride = WAVES * (STAGE == 0 ? 8 * NT : 16 * NT) / (STAGE == 0 ? 64 : 128);
  const size_t w_unit_stride = PACKED ? (size_t)kPackedStride * (size_t)nsteps * (size_t)kMxStepBytes
                                      : unit_stride_rows * (size_t)(K / 2);
  const size_t s_unit_stride = unit_stride_rows * (size_t)groups;
  constexpr int kNS = PACKED ? (STAGE == 0 ? NT / 2 : NT) : 1;  // scale words of a K step a lane loads

  // Order of the start: what memory must bring is asked for first (wavefront 0: the experts
  // of the first 64 blocks, for the run list; the others: the head of sorted_ids, which
  // they copy to the start of the operand planes, free until the first pass is staged, so
  // that the ids of the workgroup's first rows are an LDS read behind the barrier), then
  // every wavefront does the set-up that does not depend on its slice while those loads
  // are under way, then the run list and the slice.
  int* const ids_lds = reinterpret_cast<int*>(b_lds);
  const int ids_cached = min(p.num_blocks * p.block_size, nsteps * 1024);  // 4 KB of planes per K step
  constexpr int kIdsAhead = 2;  // loads of the copy a lane asks for before the set-up
  int e_first = -1;             // wavefront 0: the expert of block `lane`
  int ids_ahead[kIdsAhead];
  if constexpr (ROUTE) {
    // ---- router: a wavefront per token; the table of local experts stays in LDS ----
    const int n_flat = p.n_flat, top_k = p.top_k, T = n_flat / top_k;
    // (routed rows: at most kRouteMaxRows, a lane each: row tid)
    int my_le = -1;  // ROUTE == 2: the local expert of row tid
    if constexpr (ROUTE == 2) {  // the ids are the router's; asked for first, the tables cleared meanwhile
      if (tid < n_flat) {
        const int id = p.rt_topk_ids[tid];
        if (id >= 0 && id < p.rt_experts) {
          my_le = p.rt_expert_map != nullptr ? p.rt_expert_map[id] : id;
          if (my_le < 0 || my_le >= p.rt_local_n) my_le = -1;
        }
      }
    }
    for (int i = tid; i < (kRouteMaxRows / 64) * kRouteMaxExperts; i += 64 * WAVES) (&rt_cnt[0][0])[i] = 0;
    for (int i = tid; i < kRouteMaxRows * 8; i += 64 * WAVES) reinterpret_cast<uint32_t*>(run_ids)[i] = 0xFFFFFFFFu;
    for (int token = wave; ROUTE == 1 && token < T; token += WAVES) {  // uniform per wavefront
      int my_id;
      float my_w;
      route_token<kRoutePer>(p.rt_logits + (size_t)token * p.rt_experts, p.rt_experts, top_k,
                             p.rt_renormalize, lane, my_id, my_w);
      if (lane < top_k) {
        int le = -1;
        if (my_id >= 0 && my_id < p.rt_experts) {
          le = p.rt_expert_map != nullptr ? p.rt_expert_map[my_id] : my_id;
          if (le < 0 || le >= p.rt_local_n) le = -1;
        }
        rt_le[token * top_k + lane] = (short)le;
        if (blockIdx.x == 0) {
          p.rt_topk_ids[(size_t)token * top_k + lane] = my_id;
          p.rt_topk_w[(size_t)token * top_k + lane] = my_w;
        }
      }
    }
    __syncthreads();  // (the tables are cleared; ROUTE == 1: rt_le is written)
    // ---- every routed row among the rows of its expert: lane = row tid; the lanes of a
    // wavefront with the same expert are found with a ballot per bit of the expert's
    // number, the row's rank among them is the count of the lower lanes, and their number
    // goes to the wavefront's line of rt_cnt ----
    if constexpr (ROUTE == 1) my_le = tid < n_flat ? (int)rt_le[tid] : -1;
    int my_rank = 0;
    if (tid < kRouteMaxRows) {  // uniform per wavefront
      unsigned long long same = __ballot(my_le >= 0);
#pragma unroll
      for (int b = 0; b < 8; ++b) {  // kRouteMaxExperts = 2^8
        const unsigned long long set = __ballot(((my_le >> b) & 1) != 0);
        same &= ((my_le >> b) & 1) != 0 ? set : ~set;
      }
      my_rank = (int)__popcll(same & ((1ull << lane) - 1ull));
      if (my_le >= 0 && my_rank == 0) rt_cnt[tid >> 6][my_le] = (int)__popcll(same);
    }
    __syncthreads();
    // ---- first block of every expert (wavefront 0: a scan of the blocks, 64 experts a trip) ----
    if (wave == 0) {
      int blocks = 0;
      for (int base = 0; base < p.rt_local_n; base += 64) {
        const int e = base + lane;
        int c = 0;
        if (e < p.rt_local_n) {
#pragma unroll
          for (int w = 0; w < kRouteMaxRows / 64; ++w) c += rt_cnt[w][e];
        }
        const int nb_e = (c + 15) >> 4;
        int incl = nb_e;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int y = __shfl_up(incl, d);
          if (lane >= d) incl += y;
        }
        if (e < p.rt_local_n) rt_hist[e] = blocks + incl - nb_e;  // the expert's first block
        // the runs: every block with rows, in order
        for (int b = 0; b < nb_e; ++b) {
          const int r = blocks + incl - nb_e + b;
          run_block0[r] = r;
          run_expert[r] = e;
          run_cum[r] = r + 1;
        }
        blocks += __shfl(incl, 63);
      }
      if (lane == 0) {
        rt_runs = blocks;
        pass_slow[0] = 0;
        pass_slow[1] = 0;
      }
    }
    __syncthreads();
    // ---- place of every routed row: its rank among the rows of its expert ----
    const int n_runs = rt_runs;
    if (my_le >= 0) {  // (rows in ascending order inside an expert: those of the wavefronts before, then the lower lanes)
      int rank = my_rank;
      for (int w = 0; w < (tid >> 6); ++w) rank += rt_cnt[w][my_le];
      run_ids[rt_hist[my_le] * 16 + rank] = (unsigned short)tid;
    }
    __syncthreads();
    // ---- workgroup 0: the tables for the second stage and the caller ----
    if (blockIdx.x == 0) {
      const int em = min(n_runs > 0 ? n_runs * 16 : 16, p.rt_max_em);
      if (tid == 0) *p.rt_out_em = em;
      for (int r = tid; r < p.rt_max_em; r += 64 * WAVES) {
        int id = n_flat;
        if (r < n_runs * 16 && run_ids[r] != 0xFFFF) id = run_ids[r];
        p.rt_sorted_ids[r] = id;
      }
      for (int b = tid; b < p.rt_max_em / 16; b += 64 * WAVES) p.rt_expert_ids[b] = b < n_runs ? run_expert[b] : -1;
    }
  } else if (wave == 0) {
    e_first = p.expert_ids[min(lane, p.num_blocks - 1)];
  } else {
#pragma unroll
    for (int j = 0; j < kIdsAhead; ++j)
      ids_ahead[j] = p.sorted_ids[min(tid - 64 + j * 64 * (WAVES - 1), ids_cached - 1)];
  }

  // Scale bytes of a unit: byte offset of this lane's piece j from the unit's first tile
  // (tile_row = the first weight row of the piece's tile, counted from the first tile's, as
  // unit_tiles lays them out; lanes past the end re-read the last piece).
  constexpr int kHalfTiles = NT >= 2 ? NT / 2 : 1;
  constexpr int kScMax = resident_scale_pieces(WAVES);
  int sc_piece[kScMax];
#pragma unroll
  for (int j = 0; j < kScMax; ++j) {
    const int piece = min(lane + 64 * j, NT * groups - 1);
    int t = 0;
#pragma unroll
    for (int t2 = 1; t2 < NT; ++t2)
      if (piece >= t2 * groups) t = t2;
    int tile_row = STAGE == 0 ? 0 : t * 16;
    if (STAGE == 0) {
#pragma unroll
      for (int t2 = 1; t2 < NT; ++t2)
        if (t == t2) tile_row = (t2 / kHalfTiles) * p.ncols + (t2 % kHalfTiles) * 16;
    }
    sc_piece[j] = tile_row * groups + (piece - t * groups) * 16;
  }

  static_assert(WAVES % 4 == 0, "a wavefront's pieces keep their quarter of a K step");

  if (!ROUTE && WAVES > 1 && wave != 0) {
#pragma unroll
    for (int j = 0; j < kIdsAhead; ++j) {
      const int i = tid - 64 + j * 64 * (WAVES - 1);
      if (i < ids_cached) ids_lds[i] = ids_ahead[j];
    }
    for (int i = tid - 64 + kIdsAhead * 64 * (WAVES - 1); i < ids_cached; i += 64 * (WAVES - 1))
      ids_lds[i] = p.sorted_ids[i];
  }

  // ---- list the runs (first and last block of every run, in order) ---------
  if (wave == 0) {
    const int nb = p.num_blocks;
    const int grid = (int)gridDim.x, wg = xcd_major_index((int)blockIdx.x, (int)gridDim.x);
    const unsigned long long below = (1ull << lane) - 1ull;
    // Every block with an expert is a run of its own: the blocks of an expert then go to
    // different workgroups side by side, each staging once, where a run of several blocks
    // would have every workgroup of its share stage pass after pass.  Weight of a run =
    // its 16-row tiles that hold routed rows: 1 for blocks of 16; for larger blocks the
    // tiles whose first row is routed (the rows of an expert are packed at the front of its
    // blocks; where they are not, only the balance of the split suffers: which tiles are
    // passes is decided below from all their rows).
    const int tpb = p.block_size / 16;
    int n = 0;
    int listed_weight = 0;  // weight of the runs so far
    if constexpr (ROUTE) {  // the runs are listed already: every block with rows, weight 1 each
      n = rt_runs;
      listed_weight = n;
    }
    for (int base = 0; !ROUTE && base < nb; base += 64) {
      const int b = base + lane;
      const int bc = min(b, nb - 1);
      const int e_here = base == 0 ? e_first : p.expert_ids[bc];
      int w = tpb;  // (more than 8 tiles a block: all of them)
      if (tpb > 1 && tpb <= 8) {  // uniform; loads without a branch between them: one round trip
        w = 0;
#pragma unroll
        for (int jt = 0; jt < 8; ++jt) {
          const int id = p.sorted_ids[(size_t)(bc * tpb + min(jt, tpb - 1)) * 16];
          w += (jt < tpb && id >= 0 && id < p.n_flat) ? 1 : 0;
        }
        w = max(w, 1);
      }
      const int e = b < nb ? e_here : -1;
      const bool run = e >= 0;
      const unsigned long long mr = __ballot(run);
      int cum = run ? w : 0;  // inclusive prefix of the weights over the lanes
      if (tpb > 1) {
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int y = __shfl_up(cum, d);
          if (lane >= d) cum += y;
        }
      } else {
        cum = (int)__popcll(mr & below) + (run ? 1 : 0);
      }
      if (run) {
        const int idx = n + (int)__popcll(mr & below);
        if (idx < kMaxRuns) {
          run_block0[idx] = b;
          run_expert[idx] = e;
          run_cum[idx] = listed_weight + cum;
        }
      }
      n += (int)__popcll(mr);
      listed_weight += tpb > 1 ? __shfl(cum, 63) : (int)__popcll(mr);
    }
    n = n < kMaxRuns ? n : kMaxRuns;
    if (lane == 0) {
      pass_slow[0] = 0;
      pass_slow[1] = 0;
    }
    // ---- this workgroup's slice --------------------------------------------
    // Aligned slicing gives the runs up to and including r the first
    // floor(grid * (their weight) / (all weight)) workgroups (run_cum = the weights
    // summed).  A lane per run, and ballots instead of reductions: this wavefront is the
    // only one at work until the barrier below.
    const int total_weight = listed_weight;
    bool ok = n > 0 && n <= grid;
    int t0 = 0, t1 = 0;
    if (ok) {
      // largest (units per workgroup) x (passes) a run may have
      const int limit = (units * total_weight + grid - 1) / grid + kStagingUnits;
      int mine = -1, mine_begin = 0, mine_end = 0;  // the first run whose workgroups end past this one
      for (int base = 0; base < n; base += 64) {
        const int r = base + lane;
        const bool live = r < n;
        const int cum = live ? run_cum[r] : 0;  // written by this wavefront; LDS operations stay in order
        const int len = cum - (live && r > 0 ? run_cum[r - 1] : 0);  // the run's weight
        const int end = (int)((unsigned)(grid * cum) / (unsigned)total_weight);
        const int begin = (int)((unsigned)(grid * (cum - len)) / (unsigned)total_weight);
        bool bad = false;
        if (live) {
          bad = end <= begin;
          if (!bad) bad = (units + end - begin - 1) / (end - begin) * len > limit;
        }
        ok = ok && __ballot(bad) == 0ull;
        const unsigned long long past = __ballot(live && end > wg);
        if (mine < 0 && past != 0ull) {  // uniform
          const int l = __builtin_ctzll(past);
          mine = base + l;
          mine_begin = __builtin_amdgcn_readlane(begin, l);
          mine_end = __builtin_amdgcn_readlane(end, l);
        }
      }
      if (ok) {  // the last run ends at `grid`, so `mine` is set
        const int g = mine_end - mine_begin;
        t0 = mine * units + slice_begin(units, wg - mine_begin, g);
        t1 = mine * units + slice_begin(units, wg - mine_begin + 1, g);
      }
    }
    if (!ok && n > 0) {  // the (run, unit) space cut evenly; a slice may span runs
      t0 = slice_begin(n * units, wg, grid);
      t1 = slice_begin(n * units, wg + 1, grid);
    }
    if (lane == 0) {
      slice_sh[0] = t0;
      slice_sh[1] = t1;
    }
  }
  lds_barrier();
  const int s0 = slice_sh[0], s1 = slice_sh[1];  // n_runs * units is far below 2^31
  if (s0 >= s1) return;  // uniform over the workgroup

  struct Stage {
    u32x4 w[NT];
    uint32_t s[kNS];  // PACKED: the scale bytes of the step (tile t: word t % kNS, byte shift[t] / 8)
  };
  int pass_no = 0;

  // Segments of the slice: the units [u0, u1) of run r.  K split: at most WAVES / 2 units
  // at a time, each shared by WAVES / (u1 - u0) wavefronts (ks_n of them, wavefront
  // my_u + c * n_seg the c-th part of K: steps [k_begin, k_end)), summed through LDS.
  for (int sl = s0; sl < s1;) {
    const int r = sl / units;
    const int base_slot = r * units;
    const int u0 = sl - base_slot;
    int u1_ = min(s1, base_slot + units) - base_slot;
    if constexpr (KSPLIT) u1_ = min(u1_, u0 + WAVES / 2);
    const int u1 = u1_;
    sl = base_slot + u1;
    const int b0 = run_block0[r];
    const int run_blocks = 1;  // every block is a run of its own
    const int e = run_expert[r];
    const int run_row0 = b0 * p.block_size;
    const int run_tiles = run_blocks * (p.block_size / 16);
    // units of this wavefront in the segment: first, first + WAVES, ...
    int first_ = u0 + wave;
    int n_my_ = first_ < u1 ? (u1 - first_ + WAVES - 1) / WAVES : 0;
    int n_seg = 1, ks_n = 1, my_c = 0, k_begin_ = 0, k_end_ = nsteps;
    if constexpr (KSPLIT) {
      n_seg = u1 - u0;                      // 1 .. WAVES / 2
      ks_n = min(WAVES / n_seg, nsteps);    // parts of K, every one with a step
      my_c = wave / n_seg;
      first_ = u0 + (wave - my_c * n_seg);
      n_my_ = my_c < ks_n ? 1 : 0;
      if (n_my_ > 0) {
        k_begin_ = my_c * nsteps / ks_n;
        k_end_ = (my_c + 1) * nsteps / ks_n;
      }
    }
    const int first = first_, n_my = n_my_, k_begin = k_begin_, k_end = k_end_;

    // compute-side pointers of the current unit (start: the first one)
    const uint8_t* cw[NT];
    const uint8_t* cs[NT];
    int col0[NT];
    int shift[NT];         // PACKED: where a tile's scale byte is in the step's word
    int cur_pu = 0;        // PACKED: packed unit of the unit being computed ...
    uint32_t cur_flag = 0u;  // ... and its flag (packed_unit_flag)

    // ---- load cursor: runs D steps ahead and crosses unit boundaries -----
    const uint8_t* lrow[NT];
    const uint8_t* lsc[kNS];
#pragma unroll
    for (int t = 0; t < NT; ++t) lrow[t] = nullptr;
#pragma unroll
    for (int j = 0; j < kNS; ++j) lsc[j] = nullptr;
    int ld_ks = 0;
    int ld_units = 0;  // units the cursor has not finished, the current one included
    auto issue = [&](Stage& st) {
      // lanes past the end of a partial last step re-read the last group: the
      // operand planes there are zero, so what they load does not matter
      if constexpr (PACKED) {  // (the packed form is padded to whole K steps with zero codes)
        const size_t step = (size_t)ld_ks * (size_t)kMxStepBytes;
#pragma unroll
        for (int t = 0; t < NT; ++t) st.w[t] = *reinterpret_cast<const u32x4*>(lrow[t] + step);
#pragma unroll
        for (int j = 0; j < kNS; ++j) st.s[j] = *reinterpret_cast<const uint32_t*>(lsc[j] + step);
      } else {
        const int g = min(ld_ks * 4 + lq, groups - 1);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          st.w[t] = *reinterpret_cast<const u32x4*>(lrow[t] + (size_t)g * 16);
      }
      if constexpr (KSPLIT) {
        if (++ld_ks == k_end) ld_ks = k_end - 1;  // past this wavefront's part: stay on its last step
      } else if (++ld_ks == nsteps) {  // uniform, no memory operation inside
        if (ld_units > 1) {
          --ld_units;
          ld_ks = 0;
#pragma unroll
          for (int t = 0; t < NT; ++t) lrow[t] += w_unit_stride;
          if constexpr (PACKED) {
#pragma unroll
            for (int j = 0; j < kNS; ++j) lsc[j] += w_unit_stride;
          }
        } else {
          ld_ks = nsteps - 1;  // past the last unit: stay on its last step
        }
      }
    };

    // ---- scale block of a unit: coalesced loads into registers, parked in
    // the wavefront's LDS region when the unit before it is complete --------
    // The unit's tiles are read as NT * groups 16-byte pieces, lane + 64 j the pieces of a
    // lane (sc_piece: where piece j lies from the start of the unit's first tile) and
    // parked in the same order: tile t starts at piece t * groups, which is where
    // sc_lds + t * sc_tile_bytes is.
    u32x4 scn[kScMax];
    const uint8_t* sc_unit = nullptr;  // scale bytes of the first tile of the unit being computed
    auto fetch_scales = [&](size_t ahead) {
      if constexpr (PACKED) return;
#pragma unroll
      for (int j = 0; j < kScMax; ++j)
        scn[j] = *reinterpret_cast<const u32x4*>(sc_unit + ahead + sc_piece[j]);
    };
    auto park_scales = [&]() {
      if constexpr (PACKED) return;
#pragma unroll
      for (int j = 0; j < kScMax; ++j) {
        const int piece = lane + 64 * j;
        if (piece < NT * groups) *reinterpret_cast<u32x4*>(sc_lds + piece * 16) = scn[j];
      }
    };


    // Start of a pass's weight stream: pointers of the wavefront's first unit,
    // its scale block and the first D steps.  Issued right behind the row loads
    // of the pass, so the weights are under way while the rows are split and
    // written; a wavefront without units loads the slice's first unit and drops it.
    Stage st[D];
    auto prime = [&]() {
      if constexpr (PACKED) {
        unit_tiles_packed<STAGE, NT>(p, e, n_my > 0 ? first : u0, lane, nsteps, cw, cs, shift, col0, cur_pu);
        cur_flag = packed_unit_flag(p, e, cur_pu);
#pragma unroll
        for (int j = 0; j < kNS; ++j) lsc[j] = cs[j];
      } else {
        unit_tiles<STAGE, NT>(p, e, n_my > 0 ? first : u0, ln, cw, cs, col0);
        sc_unit = cs[0] - (size_t)ln * groups;
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) lrow[t] = cw[t];
      ld_ks = KSPLIT ? k_begin : 0;
      ld_units = max(n_my, 1);
      fetch_scales(0);
#pragma unroll
      for (int i = 0; i < D; ++i) issue(st[i]);
    };

    // Passes of 16 rows, four at a time: one load brings the ids of 64 rows,
    // and a pass none of whose rows is routed is skipped.
    for (int tile0 = 0; tile0 < run_tiles; tile0 += 4) {
      int fl = -1;
      if (tile0 * 16 + lane < run_tiles * 16) {
        const int at = run_row0 + tile0 * 16 + lane;
        // uniform: the first rows a workgroup stages come from the copy in LDS
        if constexpr (ROUTE) {
          const int x = run_ids[at];  // (a run is a block of 16 rows: index = the sorted row)
          fl = x == 0xFFFF ? -1 : x;
        } else if (pass_no == 0 && run_row0 + tile0 * 16 + 64 <= ids_cached) {
          fl = ids_lds[at];
        } else {
          fl = p.sorted_ids[at];
        }
      }
      if (fl < 0 || fl >= p.n_flat) fl = -1;
      const unsigned long long routed = __ballot(fl >= 0);
      for (int tt = 0; tt < 4; ++tt) {
        if (((routed >> (16 * tt)) & 0xFFFFull) == 0ull) continue;  // same in every wavefront
        const int tile = tile0 + tt;
        const int my_flat = __shfl(fl, tt * 16 + ln);         // row of this lane's outputs
        const int st_flat = __shfl(fl, tt * 16 + (lane >> 2));  // row this lane stages
        int flat4[4];  // second stage: the rows 4 lq + r of this lane's outputs (epilogue_rows)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) flat4[r4] = STAGE == 1 ? __shfl(fl, tt * 16 + 4 * lq + r4) : -1;
        float w4[4] = {0.f, 0.f, 0.f, 0.f};
        if constexpr (STAGE == 1) rows_weights(p, flat4, w4);
        const int srow = run_row0 + tile * 16 + ln;
        const int flag = pass_no & 1;
        ++pass_no;

        // ---- stage the 16 rows, all of K, as MFMA operands --------------------
        // Lane (j, d) = (lane / 4, lane % 4) takes the 8 values k = 32 g + 8 d ..
        // of row j for group g = pq; the four lanes of a group share the block
        // scale.  All the loads of a lane (up to kBatch) are in flight together.
        // Order of issue: the row pieces that the first D K steps need, then the
        // first D steps of the weight stream (every wavefront, with or without
        // units: no branch between the loads, so that the waits below count them
        // exactly), then the rest of the rows.  The weights are so asked for as early
        // as the order of the data allows, and both they and the later row pieces
        // stay in flight while the first pieces are split and written.
        constexpr int kBatch = resident_batch(WAVES, WIDEK);  // pieces per lane, all of K in one batch
        // pieces of a lane that K steps [0, D) need (K split: all, every part starts at once)
        constexpr int kFirst = KSPLIT ? kBatch : ((D * 4 + WAVES - 1) / WAVES < kBatch ? (D * 4 + WAVES - 1) / WAVES : kBatch);
        const int n_pieces = (nsteps * 4 + WAVES - 1) / WAVES;  // the launcher keeps it <= kBatch
        // What depends on the wavefront and the lane alone is formed here, from values the
        // compiler cannot see through, and not once in front of the loops over segments and
        // passes: hoisted there, the dozens of piece predicates, plane addresses and row
        // addresses would live through the whole kernel, beyond what the register file
        // holds, and their reloads from the spill area would each wait for every load in
        // flight.
        int wave_l = wave;
        __asm__ volatile("" : "+s"(wave_l));
        int lane_l = lane;
        __asm__ volatile("" : "+v"(lane_l));
        // Staging: a wavefront takes the groups wave, wave + WAVES, ... (its pieces 0, 1, ...).
        const int my_groups = (groups - wave_l + WAVES - 1) / WAVES;      // pieces with values of the row
        const int my_pieces = (nsteps * 4 - wave_l + WAVES - 1) / WAVES;  // ... and those of the zero padding
        // where lane (row lane / 4, eighth lane % 4) writes piece 0: the leading plane
        // (the remainder plane is 2 KB on) and the block scale byte
        uint8_t* const plane0 =
            reinterpret_cast<uint8_t*>(b_lds) +
            (size_t)((((wave_l >> 2) * 4 + ((wave_l >> 1) & 1)) * 64 + ((wave_l & 1) * 2 + ((lane_l & 3) >> 1)) * 16 +
                      (lane_l >> 2)) * 16 + (lane_l & 1) * 8);
        uint8_t* const bsc0 = bsc_lds + (wave_l >> 2) * 64 + (wave_l & 3) * 16 + (lane_l >> 2);
        const int sd = lane_l & 3;
        const int sj = lane_l >> 2;
        // The row pieces of a lane: one 32-bit offset per lane from the uniform base (the row,
        // the wavefront's group and the lane's eighth of it) and a uniform offset per piece,
        // so that the dozen loads share one address register.  A lane without a row, or a
        // wavefront without a group, reads the first bytes of the first row instead.
        const bool has_row = st_flat >= 0 && my_groups > 0;
        const uint32_t row_off =
            has_row ? ((uint32_t)(STAGE == 0 ? st_flat / p.top_k : run_row0 + tile * 16 + sj) * (uint32_t)p.a_stride +
                       (uint32_t)(wave_l * 32 + sd * 8)) * 2u
                    : 0u;
        const char* const a_base = reinterpret_cast<const char*>(p.A);
        auto load_piece = [&](int it) {
          // branch-free: an invalid piece reads piece 0 again
          const uint32_t piece_off = it < my_groups ? (uint32_t)(it * WAVES * 64) : 0u;  // uniform
          return *reinterpret_cast<const u32x4*>(a_base + piece_off + row_off);
        };
        u32x4 v[kBatch];
#pragma unroll
        for (int it = 0; it < kFirst; ++it) v[it] = load_piece(it);
        __builtin_amdgcn_sched_barrier(0);  // (the order of issue is the point)
        prime();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int it = kFirst; it < kBatch; ++it) v[it] = load_piece(it);
        __builtin_amdgcn_sched_barrier(0);
        // Block scale byte of a piece (0 = outside the fast path's range).
        auto block_scale = [&](const u32x4& x) -> uint32_t {
          uint32_t emax = bf16x8_max_exponent(x);
          emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0xB1, 0xF, 0xF, true));
          emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0x4E, 0xF, 0xF, true));
          if (emax == 0u) return 127u;  // a block of zeros (or bf16 subnormals, taken as zero)
          const uint32_t sb = emax - 7u;
          return (sb < kScaleLo || sb > kScaleHi) ? 0u : sb;
        };
        // Split and write the pieces [staged, upto) of this lane.  Piece `it` of
        // wavefront w is group w + it * WAVES, so once every wavefront has
        // written `n` pieces the K steps below n * WAVES / 4 are complete.  A block
        // outside the fast path's range (checked here, as the pieces arrive) marks the
        // pass for the exact path: the mark is complete once every piece is written, which
        // is before the first unit of any wavefront is (its last K step needs the last
        // pieces), so nothing of a marked pass is stored by the fast path.
        int staged = 0;
        auto write_rows = [&](int upto) {
          bool slow = false;
#pragma unroll
          for (int it = 0; it < kBatch; ++it) {
            if (it >= staged && it < upto && it < my_pieces) {
              u32x4 x = v[it];
              if (!(it < my_groups && st_flat >= 0)) x = u32x4{0u, 0u, 0u, 0u};
              uint32_t sb = block_scale(x);
              if (sb == 0u) {  // the pass takes the exact path; keep the bytes defined
                slow = true;
                sb = 127u;
              }
              uint2 hi, lo;
              split_bf16x8(x, sb, hi, lo);
              // piece `it` is group wave + it * WAVES: K step (wave / 4) + it * (WAVES / 4),
              // quarter wave % 4 of it, so its places are those of piece 0 plus constants
              uint8_t* plane = plane0 + it * (WAVES / 4) * 4096;
              *reinterpret_cast<uint2*>(plane) = hi;
              *reinterpret_cast<uint2*>(plane + 2 * 64 * 16) = lo;
              if (sd == 0) bsc0[it * (WAVES / 4) * 64] = (uint8_t)sb;
            }
          }
          if (slow) pass_slow[flag] = 1;
          staged = upto;
        };
        // pieces every wavefront must have written before K steps [0, steps) can run
        auto pieces_for = [&](int steps) { return min(n_pieces, (steps * 4 + WAVES - 1) / WAVES); };

        lds_barrier();  // the previous pass is done with the planes and with its flag
        // The rows are staged in K order, a few K steps ahead of the first unit's
        // arithmetic, with a barrier after each portion: the weight stream starts
        // after the first portion and the rest of the splitting overlaps it.
        write_rows(KSPLIT ? n_pieces : pieces_for(min(nsteps, D)));  // (K split: every part starts at once)
        if (n_my > 0) {
          park_scales();
          if (n_my > 1) fetch_scales(s_unit_stride);
        }
        lds_barrier();
        if (tid == 0) pass_slow[flag ^ 1] = 0;  // for the next pass; its last reader is behind us

        f32x4 acc[NT];
        unsigned long long redo = 0ull;  // units (bit = index among this wavefront's) to redo
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        uint32_t bad = 0u;

        auto compute = [&](const Stage& sg, int ks) {
          const int g = min(ks * 4 + lq, groups - 1);
          int sa[NT];
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            if constexpr (PACKED) {
              sa[t] = (int)((sg.s[t % kNS] >> shift[t]) & 0xFFu);
            } else {
              const uint32_t sb = sc_lds[t * sc_tile_bytes + ln * groups + g];
              bad |= (uint32_t)((sb - kScaleLo) > (kScaleHi - kScaleLo));
              bad |= fp4x8_nonfinite(sg.w[t][0]) | fp4x8_nonfinite(sg.w[t][1]) |
                     fp4x8_nonfinite(sg.w[t][2]) | fp4x8_nonfinite(sg.w[t][3]);
              sa[t] = (int)sb - 1;
            }
          }
          const int sbh = bsc_lds[ks * 64 + lane];
          const int sbl = sbh - 4;
          const u32x4 h0 = b_lds[(ks * 4 + 0) * 64 + lane], h1 = b_lds[(ks * 4 + 1) * 64 + lane];
          const u32x4 l0 = b_lds[(ks * 4 + 2) * 64 + lane], l1 = b_lds[(ks * 4 + 3) * 64 + lane];
          const i32x8 bh = fp8_operand(h0, h1);
          const i32x8 bl = fp8_operand(l0, l1);
          i32x8 wa[NT];
#pragma unroll
          for (int t = 0; t < NT; ++t) wa[t] = PACKED ? fp4_operand_packed(sg.w[t]) : fp4_operand(sg.w[t]);
          // the two MFMAs of an accumulator are kept NT instructions apart
          // (second stage: the rows as the first operand, for epilogue_rows)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = STAGE == 1 ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bh, wa[t], acc[t], 0, 4, 0,
                                                                                   sbh, 0, sa[t])
                                : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bh, acc[t], 4, 0, 0,
                                                                                   sa[t], 0, sbh);
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = STAGE == 1 ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bl, wa[t], acc[t], 0, 4, 0,
                                                                                   sbl, 0, sa[t])
                                : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bl, acc[t], 4, 0, 0,
                                                                                   sa[t], 0, sbl);
        };

        if constexpr (KSPLIT) {
          // All the rows were written before the barrier above, so the mark is complete.
          const bool slow_pass = pass_slow[flag] != 0;
          if (slow_pass) {
            redo = n_my >= 64 ? ~0ull : (1ull << n_my) - 1ull;
            if (my_c > 0) redo = 0ull;  // the unit's first wavefront redoes all of it
          } else {
            // this wavefront's part of K (none: a wavefront left over), then the parts of
            // a unit summed in order by its first wavefront; every wavefront keeps the barriers
            const int my_steps = n_my > 0 ? k_end - k_begin : 0;
            for (int f0 = 0; f0 < my_steps; f0 += D) {
#pragma unroll
              for (int i = 0; i < D; ++i) {
                if (f0 + i < my_steps) compute(st[i], k_begin + f0 + i);  // uniform
                issue(st[i]);
              }
            }
            __syncthreads();  // every wavefront is done with the operand planes: they hold the sums now
            f32x4* const part = reinterpret_cast<f32x4*>(b_lds);
            bool any_bad = __ballot(bad != 0u) != 0ull;
            if (n_my > 0 && my_c > 0) {
#pragma unroll
              for (int t = 0; t < NT; ++t) part[(wave * NT + t) * 64 + lane] = acc[t];
              if (lane == 0) ks_bad[wave] = any_bad ? 1 : 0;
            }
            __syncthreads();
            if (n_my > 0 && my_c == 0) {
              for (int c = 1; c < ks_n; ++c) {
                const int w2 = wave + c * n_seg;
#pragma unroll
                for (int t = 0; t < NT; ++t) acc[t] += part[(w2 * NT + t) * 64 + lane];
                any_bad |= ks_bad[w2] != 0;
              }
              if (any_bad || (PACKED && cur_flag != 0u))
                redo = 1ull;
              else if (STAGE == 1)
                epilogue_rows<NT>(p, e, acc, col0, flat4, w4, run_row0 + tile * 16, lane);
              else if (my_flat >= 0)
                epilogue_tile<STAGE, NT>(p, e, acc, col0, my_flat, srow, lq);
            }
          }
        } else {
          if (n_my == 0) {
            // no stream here: finish the staging in step with the other wavefronts
            for (int f0 = D; staged < n_pieces; f0 += D) {
              write_rows(pieces_for(min(nsteps, f0 + D)));
              lds_barrier();
            }
            continue;
          }
          const int total_steps = n_my * nsteps;
          int cks = 0;    // K step of the unit being computed
          int cunit = 0;  // its index among this wavefront's units
          for (int f0 = 0; f0 < total_steps; f0 += D) {
            if (f0 > 0 && staged < n_pieces) {  // uniform, and the same in every wavefront
              write_rows(pieces_for(min(nsteps, f0 + D)));
              lds_barrier();
            }
#pragma unroll
            for (int i = 0; i < D; ++i) {
              if (f0 + i < total_steps) {  // uniform
                compute(st[i], cks);
                if (++cks == nsteps) {
                  // ---- the unit is complete ---------------------------------
                  // (every piece of the rows was written, and its barrier passed, before this
                  // unit's last K step could run: the pass's mark is complete.)  A unit of a
                  // marked pass, or one that met a code or scale outside the fast path's
                  // domain, is redone after the stream, so the hot loop stays small
                  if (__ballot(bad != 0u) != 0ull || pass_slow[flag] != 0 || (PACKED && cur_flag != 0u))
                    redo |= 1ull << cunit;
                  else if (STAGE == 1)
                    epilogue_rows<NT>(p, e, acc, col0, flat4, w4, run_row0 + tile * 16, lane);
                  else if (my_flat >= 0)
                    epilogue_tile<STAGE, NT>(p, e, acc, col0, my_flat, srow, lq);
                  if (++cunit < n_my) {
                    park_scales();
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                      cw[t] += w_unit_stride;
                      cs[t] += PACKED ? w_unit_stride : s_unit_stride;
                      col0[t] += WAVES * (STAGE == 0 ? 8 * NT : 16 * NT);
                    }
                    if constexpr (PACKED) {
                      cur_pu += kPackedStride;
                      cur_flag = packed_unit_flag(p, e, cur_pu);
                    } else {
                      sc_unit += s_unit_stride;
                      if (cunit + 1 < n_my) fetch_scales(s_unit_stride);
                    }
                  }
                  cks = 0;
                  bad = 0u;
#pragma unroll
                  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
              }
              issue(st[i]);
            }
          }
        }

        // ---- reference-exact pass over the units the fast path could not take
        if (redo != 0ull) {
          const uint16_t* a_row = nullptr;
          if (my_flat >= 0)
            a_row = p.A + (size_t)(STAGE == 0 ? my_flat / p.top_k : srow) * (size_t)p.a_stride;
          while (redo != 0ull) {
            const int idx = __builtin_ctzll(redo);
            redo &= redo - 1ull;
            if constexpr (PACKED) {
              unit_tiles_packed<STAGE, NT>(p, e, first + idx * WAVES, lane, nsteps, cw, cs, shift, col0, cur_pu);
              exact_unit_packed<NT, STAGE == 1>(cw, cs, shift, packed_unit_flag(p, e, cur_pu) != 0u, a_row, K, lane, acc);
            } else {
              unit_tiles<STAGE, NT>(p, e, first + idx * WAVES, ln, cw, cs, col0);
              exact_unit_global<NT, STAGE == 1>(cw, cs, a_row, K, lane, acc);
            }
            if (STAGE == 1) epilogue_rows<NT>(p, e, acc, col0, flat4, w4, run_row0 + tile * 16, lane);
            else if (my_flat >= 0) epilogue_tile<STAGE, NT>(p, e, acc, col0, my_flat, srow, lq);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Decode kernel, chunked form: the prepacked weights, rows of any K, and one or two 16-row
// tiles of an expert a pass over its weights (blocks of 16 MT rows).
//
// The resident kernel above keeps the rows of a pass in LDS for all of K, which bounds K
// (4096 values) and the rows (16).  Here the rows are in LDS a chunk of kChunkSteps K steps
// at a time, twice over (the chunk being multiplied and the next one, written while the
// first runs), and a wavefront keeps the sums of all its units of a segment in registers
// across the chunks: per chunk it walks its units' K steps of that chunk, one unit after
// the other, as one stream of loads (D steps in flight, the cursor crossing from unit to
// unit and from chunk to chunk), with one workgroup barrier a chunk.  A segment is at most
// kChunkWaves x chunked_max_units units of one run; a slice longer than that stages its rows again
// per segment (a few per cent of the segment's weight bytes).  With MT = 2 every weight
// register is multiplied with both row tiles, so an expert with 17 to 32 rows costs one
// pass over its weights instead of two (a tile without a routed row is skipped).
// Work split, arithmetic, the exact path and the epilogue are the resident kernel's.
// ---------------------------------------------------------------------------
constexpr int kChunkWaves = 8;
constexpr int kChunkSteps = 8;
// Units of a wavefront in a segment: their sums (4 registers per tile of weights and of
// rows) must leave room for the weight steps in flight and a chunk's row pieces; a kernel
// that spills pays for every reload with a wait for all its loads in flight.
__host__ __device__ constexpr int chunked_max_units(int nt, int mt) { return (mt == 2 ? 12 : 16) / nt; }
__host__ __device__ constexpr size_t chunked_lds_bytes(int mt) {
  return (size_t)2 * kChunkSteps * (size_t)mt * (4096 + 64);
}

// ONE: rows of K <= 128 x 2 kChunkSteps, which are one chunk (the two buffers as one):
// nothing to keep across chunks, so a wavefront walks its units one after the other as the
// resident kernel does, every unit's epilogue under the loads of the next (where all
// epilogues of a segment come after its stream, the second stage's atomic additions of all
// workgroups fall together, with no load in flight).
template <int STAGE, int NT, int D, int MT, bool ONE = false>
__global__ __launch_bounds__(64 * kChunkWaves) void stream_chunked_kernel(GemmArgs p) {
  constexpr int WAVES = kChunkWaves, KC = ONE ? 2 * kChunkSteps : kChunkSteps;
  constexpr int kMaxU = ONE ? 32 : chunked_max_units(NT, MT);  // units of a wavefront in a segment
  constexpr int kPieces = KC * 4 / WAVES;  // 16-byte row pieces of a lane per tile and chunk
  static_assert(KC % D == 0 && (KC * 4) % WAVES == 0, "whole rounds of the pipeline and of the staging per chunk");
  static_assert((WAVES * (STAGE == 0 ? 8 * NT : 16 * NT)) % (STAGE == 0 ? 64 : 128) == 0,
                "a wavefront's consecutive units are whole packed units apart");
  extern __shared__ u32x4 b_lds[];  // [2][KC][MT][2 terms][2 halves][64] operand planes, then the block scales
  __shared__ int run_block0[kMaxRuns];
  __shared__ int run_expert[kMaxRuns];
  __shared__ int n_runs_sh;
  __shared__ int pass_slow[2];
  if (STAGE == 0) clear_out_share<64 * WAVES>(p);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15;
  const int lq = lane >> 4;

  const int K = p.K;
  const int groups = K / 32;
  const int nsteps = (groups + 3) / 4;
  const int nchunks = (nsteps + KC - 1) / KC;
  const int units = STAGE == 0 ? p.ncols / (8 * NT) : p.ncols / (16 * NT);
  uint8_t* const bsc_lds = reinterpret_cast<uint8_t*>(b_lds + (size_t)(ONE ? 1 : 2) * KC * MT * 256);  // [2][KC][MT][64]
  constexpr int kPackedStride = WAVES * (STAGE == 0 ? 8 * NT : 16 * NT) / (STAGE == 0 ? 64 : 128);
  const size_t w_unit_stride = (size_t)kPackedStride * (size_t)nsteps * (size_t)kMxStepBytes;
  constexpr int kNS = STAGE == 0 ? NT / 2 : NT;  // scale words of a K step a lane loads

  // ---- the runs: every block with an expert, in order (a pass each) ----
  if (wave == 0) {
    const int nb = p.num_blocks;
    const unsigned long long below = (1ull << lane) - 1ull;
    int n = 0;
    for (int base = 0; base < nb; base += 64) {
      const int b = base + lane;
      const int e = b < nb ? p.expert_ids[b] : -1;
      const unsigned long long mr = __ballot(e >= 0);
      if (e >= 0) {
        const int idx = n + (int)__popcll(mr & below);
        if (idx < kMaxRuns) {
          run_block0[idx] = b;
          run_expert[idx] = e;
        }
      }
      n += (int)__popcll(mr);
    }
    if (lane == 0) {
      n_runs_sh = n < kMaxRuns ? n : kMaxRuns;
      pass_slow[0] = 0;
      pass_slow[1] = 0;
    }
  }
  lds_barrier();
  // ---- this workgroup's slice of the (run, unit) space: every run workgroups of its own
  // where that leaves them balanced (no slice then stages two runs), else cut evenly ----
  int s0 = 0, s1 = 0;
  {
    const int n = n_runs_sh;
    const int grid = (int)gridDim.x, wg = xcd_major_index((int)blockIdx.x, (int)gridDim.x);
    if (n > 0) {
      bool aligned = n <= grid;
      if (aligned) {
        const int limit = (units * n + grid - 1) / grid + kStagingUnits;
        const int g_min = grid / n;
        aligned = (units + g_min - 1) / g_min <= limit;
      }
      if (aligned) {  // run r has workgroups [grid r / n, grid (r + 1) / n)
        const int r = ((wg + 1) * n + grid - 1) / grid - 1;
        const int begin = (int)((unsigned)(grid * r) / (unsigned)n);
        const int end = (int)((unsigned)(grid * (r + 1)) / (unsigned)n);
        s0 = r * units + slice_begin(units, wg - begin, end - begin);
        s1 = r * units + slice_begin(units, wg - begin + 1, end - begin);
      } else {
        s0 = slice_begin(n * units, wg, grid);
        s1 = slice_begin(n * units, wg + 1, grid);
      }
    }
  }
  if (s0 >= s1) return;  // uniform over the workgroup

  struct Stage {
    u32x4 w[NT];
    uint32_t s[kNS];
  };
  int seg_no = 0;
  // what depends on the lane alone: where it writes a row piece and which group it stages
  const int sd = lane & 3;   // eighth of the group of 32
  const int sj = lane >> 2;  // row of the tile
  const int g4 = wave & 3;   // the wavefront's group within a K step (piece `it`: step (wave >> 2) + 2 it)
  const int plane_lane = (((g4 >> 1) * 64 + ((g4 & 1) * 2 + (sd >> 1)) * 16 + sj) * 16) + (sd & 1) * 8;

  for (int sl = s0; sl < s1;) {
    const int r = sl / units;
    const int base_slot = r * units;
    const int u0 = sl - base_slot;
    const int u1 = min(min(s1, base_slot + units) - base_slot, u0 + WAVES * kMaxU);
    sl = base_slot + u1;
    const int e = run_expert[r];
    const int run_row0 = run_block0[r] * p.block_size;  // (block_size = 16 MT)
    const int first = u0 + wave;
    const int n_my = first < u1 ? (u1 - first + WAVES - 1) / WAVES : 0;
    const int flag = seg_no & 1;
    ++seg_no;

    // ---- the rows of the run ----
    int fl = -1;
    if (lane < 16 * MT) fl = p.sorted_ids[run_row0 + lane];
    if (fl < 0 || fl >= p.n_flat) fl = -1;
    const unsigned long long routed = __ballot(fl >= 0);
    const bool live1 = MT > 1 && ((routed >> 16) & 0xFFFFull) != 0ull;  // the second tile has a routed row
    int my_flat[MT], st_flat[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      my_flat[mt] = __shfl(fl, mt * 16 + ln);   // row of this lane's outputs
      st_flat[mt] = __shfl(fl, mt * 16 + sj);   // row this lane stages
    }
    int flat4[MT][4];  // second stage: the rows 4 lq + r of this lane's outputs (epilogue_rows)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) flat4[mt][r4] = STAGE == 1 ? __shfl(fl, mt * 16 + 4 * lq + r4) : -1;
    float w4[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) w4[mt][r4] = 0.f;
      if constexpr (STAGE == 1) rows_weights(p, flat4[mt], w4[mt]);
    }
    uint32_t row_off[MT];  // bytes from A to the lane's eighth of the wavefront's first group
    bool has_row[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      has_row[mt] = st_flat[mt] >= 0;
      row_off[mt] = has_row[mt]
                        ? ((uint32_t)(STAGE == 0 ? st_flat[mt] / p.top_k : run_row0 + mt * 16 + sj) * (uint32_t)p.a_stride +
                           (uint32_t)(wave * 32 + sd * 8)) * 2u
                        : 0u;
    }
    const char* const a_base = reinterpret_cast<const char*>(p.A);
    u32x4 v[MT * kPieces];
    // piece (mt, it) of chunk c: group c KC 4 + wave + it WAVES of tile mt's rows
    auto load_rows = [&](int c) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
          const int gi = c * (KC * 4) + wave + it * WAVES;  // uniform
          const uint32_t off = gi < groups ? (uint32_t)((c * (KC * 4) + it * WAVES) * 64) + row_off[mt] : 0u;
          v[mt * kPieces + it] = *reinterpret_cast<const u32x4*>(a_base + off);
        }
      }
    };
    auto block_scale = [&](const u32x4& x) -> uint32_t {
      uint32_t emax = bf16x8_max_exponent(x);
      emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0xB1, 0xF, 0xF, true));
      emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0x4E, 0xF, 0xF, true));
      if (emax == 0u) return 127u;
      const uint32_t sb = emax - 7u;
      return (sb < kScaleLo || sb > kScaleHi) ? 0u : sb;
    };
    // split the pieces of chunk c and write them to buffer `buf`
    auto write_rows = [&](int c, int buf) {
      bool slow = false;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt > 0 && !live1) continue;  // uniform
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
          const int gi = c * (KC * 4) + wave + it * WAVES;
          u32x4 x = v[mt * kPieces + it];
          if (!(gi < groups && has_row[mt])) x = u32x4{0u, 0u, 0u, 0u};
          uint32_t sb = block_scale(x);
          if (sb == 0u) {
            slow = true;
            sb = 127u;
          }
          uint2 hi, lo;
          split_bf16x8(x, sb, hi, lo);
          const int ksl = (wave >> 2) + it * (WAVES / 4);  // step of the chunk
          const int slot = (buf * KC + ksl) * MT + mt;
          uint8_t* plane = reinterpret_cast<uint8_t*>(b_lds) + (size_t)slot * 4096 + plane_lane;
          *reinterpret_cast<uint2*>(plane) = hi;
          *reinterpret_cast<uint2*>(plane + 2 * 64 * 16) = lo;
          if (sd == 0) bsc_lds[slot * 64 + g4 * 16 + sj] = (uint8_t)sb;
        }
      }
      if (slow) pass_slow[flag] = 1;
    };

    // ---- the weight stream's cursor: chunk by chunk, within a chunk unit by unit ----
    const uint8_t* cw[NT];
    const uint8_t* cs[NT];
    int col0[NT];
    int shift[NT];
    int pu0 = 0;
    unit_tiles_packed<STAGE, NT>(p, e, n_my > 0 ? first : u0, lane, nsteps, cw, cs, shift, col0, pu0);
    const uint8_t* lrow[NT];
    const uint8_t* lsc[kNS];
#pragma unroll
    for (int t = 0; t < NT; ++t) lrow[t] = cw[t];
#pragma unroll
    for (int j = 0; j < kNS; ++j) lsc[j] = cs[j];
    int ld_i = 0;           // position in the current (unit, chunk): 0 .. its steps rounded up to D
    int ld_u = n_my;        // units of the chunk the cursor has not finished
    int ld_k0 = 0;          // first step of the cursor's chunk
    int ld_cs = min(KC, nsteps);  // its steps
    const size_t rewind = (size_t)(n_my > 0 ? n_my - 1 : 0) * w_unit_stride;
    auto issue = [&](Stage& st) {
      const size_t step = (size_t)(ld_k0 + min(ld_i, ld_cs - 1)) * (size_t)kMxStepBytes;
#pragma unroll
      for (int t = 0; t < NT; ++t) st.w[t] = *reinterpret_cast<const u32x4*>(lrow[t] + step);
#pragma unroll
      for (int j = 0; j < kNS; ++j) st.s[j] = *reinterpret_cast<const uint32_t*>(lsc[j] + step);
      if (++ld_i >= ((ld_cs + D - 1) / D) * D) {  // uniform, no memory operation inside
        ld_i = 0;
        if (--ld_u > 0) {
#pragma unroll
          for (int t = 0; t < NT; ++t) lrow[t] += w_unit_stride;
#pragma unroll
          for (int j = 0; j < kNS; ++j) lsc[j] += w_unit_stride;
        } else {  // back to the first unit, next chunk (past the last: the last again, dropped)
          ld_u = n_my;
#pragma unroll
          for (int t = 0; t < NT; ++t) lrow[t] -= rewind;
#pragma unroll
          for (int j = 0; j < kNS; ++j) lsc[j] -= rewind;
          if (ld_k0 + KC < nsteps) {
            ld_k0 += KC;
            ld_cs = min(KC, nsteps - ld_k0);
          }
        }
      }
    };

    lds_barrier();  // the segment before is done with the planes and with its flag
    if (tid == 0) pass_slow[flag ^ 1] = 0;  // for the next segment; its last reader is behind us
    load_rows(0);
    __builtin_amdgcn_sched_barrier(0);
    Stage st[D];
    if (n_my > 0) {
#pragma unroll
      for (int i = 0; i < D; ++i) issue(st[i]);
    }
    __builtin_amdgcn_sched_barrier(0);
    write_rows(0, 0);
    lds_barrier();

    auto compute = [&](const Stage& sg, int slot0, f32x4 (&a)[MT][NT]) {
      int sa[NT];
      i32x8 wa[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        sa[t] = (int)((sg.s[t % kNS] >> shift[t]) & 0xFFu);
        wa[t] = fp4_operand_packed(sg.w[t]);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt > 0 && !live1) continue;  // uniform
        const int slot = slot0 + mt;
        const int sbh = bsc_lds[slot * 64 + lane];
        const int sbl = sbh - 4;
        const u32x4 h0 = b_lds[(slot * 4 + 0) * 64 + lane], h1 = b_lds[(slot * 4 + 1) * 64 + lane];
        const u32x4 l0 = b_lds[(slot * 4 + 2) * 64 + lane], l1 = b_lds[(slot * 4 + 3) * 64 + lane];
        const i32x8 bh = fp8_operand(h0, h1);
        const i32x8 bl = fp8_operand(l0, l1);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          a[mt][t] = STAGE == 1
                         ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bh, wa[t], a[mt][t], 0, 4, 0, sbh, 0, sa[t])
                         : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bh, a[mt][t], 4, 0, 0, sa[t], 0, sbh);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          a[mt][t] = STAGE == 1
                         ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bl, wa[t], a[mt][t], 0, 4, 0, sbl, 0, sa[t])
                         : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bl, a[mt][t], 4, 0, 0, sa[t], 0, sbl);
      }
    };
    unsigned redo = 0u;

    if constexpr (ONE) {
      // (all rows are written, so the segment's mark is complete)
      int cur_pu = pu0;
      uint32_t cur_flag = n_my > 0 ? packed_unit_flag(p, e, cur_pu) : 0u;
      for (int j = 0; j < n_my; ++j) {
        f32x4 a1[MT][NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int t = 0; t < NT; ++t) a1[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int f0 = 0; f0 < nsteps; f0 += D) {
#pragma unroll
          for (int i = 0; i < D; ++i) {
            if (f0 + i < nsteps) compute(st[i], (f0 + i) * MT, a1);
            issue(st[i]);
          }
        }
        if (pass_slow[flag] != 0 || cur_flag != 0u) {
          redo |= 1u << j;
        } else {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (mt > 0 && !live1) continue;
            if (STAGE == 1) epilogue_rows<NT>(p, e, a1[mt], col0, flat4[mt], w4[mt], run_row0 + mt * 16, lane);
            else if (my_flat[mt] >= 0)
              epilogue_tile<STAGE, NT>(p, e, a1[mt], col0, my_flat[mt], run_row0 + mt * 16 + ln, lq);
          }
        }
        if (j + 1 < n_my) {
#pragma unroll
          for (int t = 0; t < NT; ++t) col0[t] += WAVES * (STAGE == 0 ? 8 * NT : 16 * NT);
          cur_pu += kPackedStride;
          cur_flag = packed_unit_flag(p, e, cur_pu);
        }
      }
    } else {
    f32x4 acc[kMaxU][MT][NT];
#pragma unroll
    for (int u = 0; u < kMaxU; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[u][mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int c = 0; c < nchunks; ++c) {
      const int steps = min(KC, nsteps - c * KC);
      const int buf = c & 1;
      const bool more = c + 1 < nchunks;  // uniform
      if (more) load_rows(c + 1);
#pragma unroll
      for (int u = 0; u < kMaxU; ++u) {
        if (u < n_my) {  // uniform
          for (int f0 = 0; f0 < steps; f0 += D) {
#pragma unroll
            for (int i = 0; i < D; ++i) {
              if (f0 + i < steps) compute(st[i], (buf * KC + f0 + i) * MT, acc[u]);
              issue(st[i]);
            }
          }
        }
        if (u == 0 && more) write_rows(c + 1, buf ^ 1);  // (their loads have had a unit's steps)
      }
      lds_barrier();
    }

    // ---- epilogue of every unit; those of a marked segment and the flagged ones on the exact path ----
    // (Here and not with a unit's last steps: inside the unrolled stream the epilogues cost
    // more registers than the kernel has, and every reload of a spilled one waits for all
    // the loads in flight.)
    const bool slow_seg = pass_slow[flag] != 0;
#pragma unroll
    for (int u = 0; u < kMaxU; ++u) {
      if (u < n_my) {
        int pu = 0;
        unit_tiles_packed<STAGE, NT>(p, e, first + u * WAVES, lane, nsteps, cw, cs, shift, col0, pu);
        if (slow_seg || packed_unit_flag(p, e, pu) != 0u) {
          redo |= 1u << u;
        } else {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (mt > 0 && !live1) continue;
            if (STAGE == 1) epilogue_rows<NT>(p, e, acc[u][mt], col0, flat4[mt], w4[mt], run_row0 + mt * 16, lane);
            else if (my_flat[mt] >= 0)
              epilogue_tile<STAGE, NT>(p, e, acc[u][mt], col0, my_flat[mt], run_row0 + mt * 16 + ln, lq);
          }
        }
      }
    }
    }  // (not ONE)
    while (redo != 0u) {
      const int u = __builtin_ctz(redo);
      redo &= redo - 1u;
      int pu = 0;
      unit_tiles_packed<STAGE, NT>(p, e, first + u * WAVES, lane, nsteps, cw, cs, shift, col0, pu);
      const bool raw = packed_unit_flag(p, e, pu) != 0u;
      for (int mt = 0; mt < MT; ++mt) {
        if (mt > 0 && !live1) continue;
        const int flat = mt == 0 ? my_flat[0] : my_flat[MT - 1];
        const int srow = run_row0 + mt * 16 + ln;
        const uint16_t* a_row = nullptr;
        if (flat >= 0) a_row = p.A + (size_t)(STAGE == 0 ? flat / p.top_k : srow) * (size_t)p.a_stride;
        f32x4 ax[NT];
        exact_unit_packed<NT, STAGE == 1>(cw, cs, shift, raw, a_row, K, lane, ax);
        if (STAGE == 1) {
          int f4[4];
          float wx[4];
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            f4[r4] = mt == 0 ? flat4[0][r4] : flat4[MT - 1][r4];
            wx[r4] = mt == 0 ? w4[0][r4] : w4[MT - 1][r4];
          }
          epilogue_rows<NT>(p, e, ax, col0, f4, wx, run_row0 + mt * 16, lane);
        } else if (flat >= 0) {
          epilogue_tile<STAGE, NT>(p, e, ax, col0, flat, srow, lq);
        }
      }
    }
  }
}

// Stage 0 with a workspace: 32 consecutive act columns (two 16-column tiles, first
// columns c0 and c1 = c0 + 16) of one 16-row tile as the next stage's split rows.
// a0, a1: the lane's 4 + 4 bf16 values of the two tiles (columns c0 + 4 lq .. and
// c1 + 4 lq ..), as epilogue_tile stored them; the four lanes (n, q = 0..3) of a row
// share the block.  Called by whole wavefronts (flat < 0 = padding row: takes
// part in the shuffles, stores nothing).
__device__ __forceinline__ void store_split_act(const GemmArgs& p, int c0, int c1, int flat, int srow,
                                                int lane, uint2 a0, uint2 a1) {
  const int lq = lane >> 4;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (flat >= 0) v = u32x4{a0.x, a0.y, a1.x, a1.y};
  uint32_t emax = bf16x8_max_exponent(v);
  emax = max(emax, (uint32_t)__shfl_xor((int)emax, 16));
  emax = max(emax, (uint32_t)__shfl_xor((int)emax, 32));
  uint32_t sb = emax - 7u, stored;
  if (emax == 0u) sb = 127u;
  stored = sb;
  if (emax != 0u && (sb < kScaleLo || sb > kScaleHi)) { stored = 0u; sb = 127u; }
  uint2 hi, lo;
  split_bf16x8(v, sb, hi, lo);
  if (flat >= 0) {
    const int kp = split_row_k(p.ncols);
    uint8_t* qrow = p.actq + (size_t)srow * (size_t)kp * 2;
    *reinterpret_cast<uint32_t*>(qrow + c0 + 4 * lq) = hi.x;
    *reinterpret_cast<uint32_t*>(qrow + c1 + 4 * lq) = hi.y;
    *reinterpret_cast<uint32_t*>(qrow + kp + c0 + 4 * lq) = lo.x;
    *reinterpret_cast<uint32_t*>(qrow + kp + c1 + 4 * lq) = lo.y;
    if (lq == 0)
      p.actqs[(size_t)srow * (size_t)split_scale_stride(p.ncols) + (c0 >> 5)] = (uint8_t)stored;
  }
}

// ---------------------------------------------------------------------------
// Tile kernel: the general path (prefill, large K, many rows per expert).
//
// A workgroup of 4 wavefronts computes up to 64 sorted rows of one expert
// (4 row tiles of 16) against 16 weight tiles (4 per wavefront: stage 0, two
// gate tiles and the two up tiles of the same columns; stage 1, four
// consecutive tiles), K in chunks of 512.  Per chunk: every lane loads its
// wavefront's weights for the chunk straight into MFMA operand registers
// (16 x 16 bytes) and the 16 scale bytes of its row, the workgroup splits the
// 64 x 512 activations into the two E4M3 terms and writes them to LDS as MFMA
// operands (64 KiB), and each wavefront then issues 4 steps x 4 row tiles x 4
// weight tiles x 2 terms scaled MFMAs, every LDS operand read serving four of
// them.  Two workgroups fit a compute unit (LDS and registers), so one
// workgroup's splitting and barriers overlap the other's MFMAs.
//
// grid.x = chunks of 4 wavefront units along the output columns, grid.y =
// groups of min(block_size, 64) sorted rows; a group lies inside one block,
// hence one expert.  Arithmetic, operand layouts and the exact fallback are
// those of the resident kernel above.
// ---------------------------------------------------------------------------
constexpr int kTileWaves = 4, kTileNT = 4, kTileMT = 4, kTileSteps = 4;

template <int STAGE>
__global__ __launch_bounds__(64 * kTileWaves, 2) void tile_gemm_kernel(GemmArgs p) {
  constexpr int NT = kTileNT, MT = kTileMT, S = kTileSteps;
  __shared__ u32x4 planes[S * MT * 4 * 64];  // [step][row tile][term][half][lane]
  __shared__ uint8_t bsc[S * MT * 64];       // block scale bytes, [step][row tile][lane]
  __shared__ int row_flat[MT * 16];
  __shared__ int group_slow;

  if (STAGE == 0) clear_out_share<64 * kTileWaves>(p);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15;
  const int lq = lane >> 4;

  const int K = p.K;
  const int groups = K / 32;
  const int n_chunks = (groups + 4 * S - 1) / (4 * S);
  const int units = STAGE == 0 ? p.ncols / (8 * NT) : p.ncols / (16 * NT);

  // ---- the rows of this group ------------------------------------------------
  const int group_rows = tile_group_rows(p.block_size, 16 * MT);
  const int row0 = blockIdx.y * group_rows;
  const int e = p.expert_ids[row0 / p.block_size];
  if (e < 0) return;
  if (tid < MT * 16) {
    int f = -1;
    if (tid < group_rows) {
      f = p.sorted_ids[row0 + tid];
      if (f < 0 || f >= p.n_flat) f = -1;
    }
    row_flat[tid] = f;
  }
  if (tid == 0) group_slow = 0;
  __syncthreads();
  uint32_t live = 0u;  // bit m: row tile m has a routed row
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    bool any = false;
#pragma unroll
    for (int j = 0; j < 16; ++j) any |= row_flat[m * 16 + j] >= 0;
    live |= (uint32_t)any << m;
  }
  if (live == 0u) return;  // uniform

  // ---- this wavefront's weight tiles --------------------------------------------
  const int unit = blockIdx.x * kTileWaves + wave;
  const bool has_unit = unit < units;
  const uint8_t* w_rows[NT];
  const uint8_t* s_rows[NT];
  int col0[NT];
  unit_tiles<STAGE, NT>(p, e, has_unit ? unit : 0, ln, w_rows, s_rows, col0);

  // ---- staging role: lane (row, d) = (tid / 4, tid % 4) ---------------------------
  const int sr = tid >> 2, sd = tid & 3;
  const int sflat = row_flat[sr];
  const uint16_t* src =
      p.A + (size_t)(sflat >= 0 ? (STAGE == 0 ? sflat / p.top_k : row0 + sr) : 0) * (size_t)p.a_stride;
  const int sm = sr >> 4, sn = sr & 15;

  f32x4 acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  uint32_t bad = 0u;
  bool slow = false;

#pragma unroll 1
  for (int c = 0; c < n_chunks; ++c) {
    // ---- weights of the chunk: operand registers and the rows' scale bytes -------
    u32x4 wq[S][NT];
    u32x4 scq[NT];
    const int g0 = c * 4 * S;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      // groups past K re-read the last one; the operand planes there are zero
      const int g = min(g0 + 4 * s + lq, groups - 1);
#pragma unroll
      for (int t = 0; t < NT; ++t)
        wq[s][t] = *reinterpret_cast<const u32x4*>(w_rows[t] + (size_t)g * 16);
    }
    if (g0 + 4 * S <= groups) {  // uniform
#pragma unroll
      for (int t = 0; t < NT; ++t) scq[t] = *reinterpret_cast<const u32x4*>(s_rows[t] + g0);
    } else {  // last, partial chunk: byte by byte
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
          uint32_t v = 0u;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            v |= (uint32_t)s_rows[t][min(g0 + 4 * s + q, groups - 1)] << (8 * q);
          scq[t][s] = v;
        }
      }
    }

    // ---- split the 64 x 512 activations of the chunk into LDS operands -----------
    __syncthreads();  // the previous chunk's arithmetic is done with the planes
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      u32x4 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int g = g0 + half * 8 + i;
        const bool valid = g < groups && sflat >= 0;
        v[i] = *reinterpret_cast<const u32x4*>(src + (valid ? g * 32 + sd * 8 : 0));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int b = half * 8 + i;  // block of 32 within the chunk
        const int g = g0 + b;
        if (!(g < groups && sflat >= 0)) v[i] = u32x4{0u, 0u, 0u, 0u};
        uint32_t emax = bf16x8_max_exponent(v[i]);
        emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0xB1, 0xF, 0xF, true));
        emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0x4E, 0xF, 0xF, true));
        uint32_t sb = emax - 7u;
        if (emax == 0u) sb = 127u;  // a block of zeros (or bf16 subnormals, taken as zero)
        else if (sb < kScaleLo || sb > kScaleHi) { slow = true; sb = 127u; }
        uint2 hi, lo;
        split_bf16x8(v[i], sb, hi, lo);
        const int s = b >> 2, qq = b & 3;
        const int slot = ((qq & 1) * 2 + (sd >> 1)) * 16 + sn;
        uint8_t* plane = reinterpret_cast<uint8_t*>(planes) +
                         (size_t)((((s * MT + sm) * 2) * 2 + (qq >> 1)) * 64 + slot) * 16 +
                         (sd & 1) * 8;
        *reinterpret_cast<uint2*>(plane) = hi;
        *reinterpret_cast<uint2*>(plane + 2 * 64 * 16) = lo;
        if (sd == 0) bsc[(s * MT + sm) * 64 + qq * 16 + sn] = (uint8_t)sb;
      }
    }
    __syncthreads();

    // ---- arithmetic ---------------------------------------------------------------
    if (has_unit) {
#pragma unroll
      for (int s = 0; s < S; ++s) {
        i32x8 wa[NT];
        int sa[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const uint32_t sbw = (scq[t][s] >> (8 * lq)) & 0xFFu;
          bad |= (uint32_t)((sbw - kScaleLo) > (kScaleHi - kScaleLo));
          bad |= fp4x8_nonfinite(wq[s][t][0]) | fp4x8_nonfinite(wq[s][t][1]) |
                 fp4x8_nonfinite(wq[s][t][2]) | fp4x8_nonfinite(wq[s][t][3]);
          sa[t] = (int)sbw - 1;
          wa[t] = fp4_operand(wq[s][t]);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          if (!((live >> m) & 1u)) continue;  // uniform
          const u32x4* pl = planes + (size_t)((s * MT + m) * 4) * 64 + lane;
          const u32x4 h0 = pl[0], h1 = pl[64], l0 = pl[128], l1 = pl[192];
          const int sbh = bsc[(s * MT + m) * 64 + lane];
          const int sbl = sbh - 4;
          const i32x8 bh = fp8_operand(h0, h1);
          const i32x8 bl = fp8_operand(l0, l1);
          // the two MFMAs of an accumulator are kept NT instructions apart
          // (second stage: the rows as the first operand, for epilogue_rows)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[m][t] = STAGE == 1 ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bh, wa[t], acc[m][t], 0, 4,
                                                                                      0, sbh, 0, sa[t])
                                   : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bh, acc[m][t], 4, 0,
                                                                                      0, sa[t], 0, sbh);
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[m][t] = STAGE == 1 ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bl, wa[t], acc[m][t], 0, 4,
                                                                                      0, sbl, 0, sa[t])
                                   : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa[t], bl, acc[m][t], 4, 0,
                                                                                      0, sa[t], 0, sbl);
        }
      }
    }
  }

  // ---- fall back to the exact path where the fast one was outside its domain ----
  if (slow) group_slow = 1;
  __syncthreads();
  if (!has_unit) return;
  const bool redo = group_slow != 0 || __ballot(bad != 0u) != 0ull;

  // ---- epilogue -----------------------------------------------------------------------
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (!((live >> m) & 1u)) continue;
    const int flat = row_flat[m * 16 + ln];
    const int srow = row0 + m * 16 + ln;
    if (redo) {
      const uint16_t* a_row = nullptr;
      if (flat >= 0) a_row = p.A + (size_t)(STAGE == 0 ? flat / p.top_k : srow) * (size_t)p.a_stride;
      exact_unit_global<NT, STAGE == 1>(w_rows, s_rows, a_row, K, lane, acc[m]);
    }
    if constexpr (STAGE == 1) {
      int flat4[4];
      float w4[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) flat4[r] = row_flat[m * 16 + 4 * lq + r];
      rows_weights(p, flat4, w4);
      epilogue_rows<NT>(p, e, acc[m], col0, flat4, w4, row0 + m * 16, lane);
    } else {
      uint2 packed[NT / 2] = {};
      if (flat >= 0) epilogue_tile<STAGE, NT>(p, e, acc[m], col0, flat, srow, lq, packed);
      if (p.actq != nullptr) store_split_act(p, col0[0], col0[1], flat, srow, lane, packed[0], packed[1]);
    }
  }
}

// ---------------------------------------------------------------------------
// Wide tile kernel (workspace path): up to 128 sorted rows of one expert per
// workgroup, so that the preparation of a weight tile (code points, inf/NaN and
// scale-range checks) is shared by 16 MFMAs and every LDS operand read by 8.
//
// 4 wavefronts, one per SIMD, each with the full register file: 8 row tiles x
// 4 weight tiles of accumulators.  Everything the K loop reads from global
// memory arrives in LDS by the DMA form of the global load, three K steps
// ahead, and no wavefront ever waits for a load it has just issued: the waits
// are s_waitcnt instructions with counts derived from the fixed order in which
// each wavefront issues its memory operations.
//
// Rows.  A workgroup takes a window of 128 sorted rows (block sizes that divide
// 128; otherwise one group of tile_group_rows rows) and cuts it into segments
// of consecutive blocks of one expert; each segment is one pass of the K loop.
//
// LDS (bytes):
//   row ring     3 x 32 KiB   per K step, 8 row tiles x {hi, lo} x 16 rows x 128
//                             bytes, copied from the split rows (whose zero blocks
//                             between K and the next multiple of 128 make the last,
//                             partial step an ordinary one) as whole cache lines;
//   row scales   2 x 2 KiB    16 scale bytes per row, of which a group of 3 K steps
//                             uses 12;
//   weight ring  4 x 3 x 4 KiB  per wavefront and K step, its 4 weight tiles as MFMA
//                             operands (lane order);
//   weight scales 4 x 2 x 1 KiB per wavefront, 16 scale bytes per weight row.
// One barrier per K step, before its last row tile: every wavefront first waits
// for its own row copies of the NEXT step, so after the barrier (a) that step may
// be read ahead and (b) the slot of the current step, whose last tile is already
// in registers, takes the copies of step + 3.  The weight ring is private to a
// wavefront and needs no barrier.
// ---------------------------------------------------------------------------
constexpr int kWideWaves = 4, kWideNT = 4, kWideMT = 8, kWideRing = 3;
constexpr int kWideRows = 16 * kWideMT;
constexpr int kWideStepBytes = kWideMT * 4 * 1024;
constexpr int kWideRowScales = kWideRing * kWideStepBytes;            // 2 slots x 128 rows x 16
constexpr int kWideWeights = kWideRowScales + 2 * kWideRows * 16;     // per wavefront: 3 x 4 KiB
constexpr int kWideWeightScales = kWideWeights + kWideWaves * kWideRing * 4096;  // per wavefront: 2 x 1 KiB
constexpr int kWideLdsBytes = kWideWeightScales + kWideWaves * 2 * 1024;

// Sorted rows one workgroup of the wide kernel covers.
__host__ __device__ inline int wide_window_rows(int block_size) {
  return kWideRows % block_size == 0 ? kWideRows : tile_group_rows(block_size, kWideRows);
}

template <int STAGE>
__global__ __launch_bounds__(64 * kWideWaves) void tile_wide_kernel(GemmArgs p) {
  constexpr int NT = kWideNT, MT = kWideMT, R = kWideRing;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  extern __shared__ u32x4 wide_lds[];
  __shared__ int row_flat[kWideRows];
  __shared__ int wave_valid[2];

  if (STAGE == 0) clear_out_share<64 * kWideWaves>(p);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15;
  const int lq = lane >> 4;

  const int K = p.K;
  const int Kp = split_row_k(K);
  const int groups = K / 32;
  const int nsteps = Kp / 128;
  const int units = STAGE == 0 ? p.ncols / (8 * NT) : p.ncols / (16 * NT);
  const int sstride = split_scale_stride(K);
  const int unit = blockIdx.x * kWideWaves + wave;
  const bool has_unit = unit < units;

  struct Rows {
    u32x4 h0, h1, l0, l1;
    int sb;
  };
  // Memory operations of a wavefront in K step c, in program order (all DMA; j = c % 3):
  //   0 .. 4    pieces 3 .. 7 of its row copies of step c + 2 (the slot was freed by the
  //             barrier of step c - 1);
  //   5 .. 8    its 4 weight tiles of step c + 3 (their slot was read during step c - 1);
  //   9 .. 12   j = 0 only: the weight-scale copies of the next group of three steps;
  //   -- the barrier of step c --
  //   13 .. 15  pieces 0 .. 2 of its row copies of step c + 3, into the slot just freed;
  //   16        j = 0 only: the row scales of the next group.
  // The operations before the barrier are spread over the row tiles of the step, so that
  // the memory pipe, which all four wavefronts share, is fed evenly while the MFMAs run.
  constexpr int kRowsLate = 5, kRowsEarly = 3, kWeightOps = NT;
  auto ops_before = [](int j) constexpr { return kRowsLate + kWeightOps + (j == 0 ? NT : 0); };
  auto ops_after = [](int j) constexpr { return kRowsEarly + (j == 0 ? 1 : 0); };

  auto segment = [&](const int row0, const int n_rows, const int e) {
    __syncthreads();  // the previous segment is done with row_flat and the rings
    if (tid < kWideRows) {
      int f = -1;
      if (tid < n_rows) {
        f = p.sorted_ids[row0 + tid];
        if (f < 0 || f >= p.n_flat) f = -1;
      }
      row_flat[tid] = f;
      // one past the highest routed row of this half of the window (padding may stand
      // anywhere among an expert's rows)
      const unsigned long long routed = __ballot(f >= 0);
      if (lane == 0) wave_valid[wave] = routed != 0ull ? 64 - (int)__builtin_clzll(routed) : 0;
    }
    __syncthreads();
    const int n_live = ((wave_valid[1] > 0 ? 64 + wave_valid[1] : wave_valid[0]) + 15) >> 4;
    if (n_live == 0) return;  // uniform

    const uint8_t* w_rows[NT];
    const uint8_t* s_rows[NT];
    int col0[NT];
    unit_tiles<STAGE, NT>(p, e, has_unit ? unit : 0, ln, w_rows, s_rows, col0);

    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr)wide_lds;
    const uint8_t* lds_bytes = reinterpret_cast<const uint8_t*>(wide_lds);

    // ---- row copies.  One copy instruction moves 8 rows x 128 bytes (one K step of
    // one term): whole cache lines, which the memory pipe serves three times as fast
    // as 64-byte pieces of 16 rows.  Lane (r, j) = (lane / 8, lane % 8) copies piece
    // j ^ r of row r, so that the 16-byte pieces of a row sit in LDS rotated by the
    // row and the MFMA operand reads (16 rows, one piece each) spread over the banks.
    // Wavefront w copies row tiles 2 w and 2 w + 1.
    const int cr = lane >> 3, cj = lane & 7;
    const uint8_t* cp_row[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int rh = 0; rh < 2; ++rh) {
        const int rl = (wave * 2 + i) * 16 + rh * 8 + cr;
        const int f = row_flat[rl];
        const size_t r = f >= 0 ? (size_t)(STAGE == 0 ? f / p.top_k : row0 + rl) : 0;
        cp_row[i][rh] = p.Aq + r * (size_t)(2 * Kp) + 16 * (cj ^ cr);
      }
    // row scale bytes: 16 per row from byte 12 g on (a group of 3 K steps uses 12);
    // rows 64 (wave % 2) .. + 63, twice over, so that all wavefronts issue alike
    const uint8_t* cp_scale;
    {
      const int rl = (wave & 1) * 64 + lane;
      const int f = row_flat[rl];
      const size_t r = f >= 0 ? (size_t)(STAGE == 0 ? f / p.top_k : row0 + rl) : 0;
      cp_scale = p.As + r * (size_t)sstride;
    }
    // piece j (0 .. 7) of this wavefront's row copies of a K step
    auto copy_row_piece = [&](int step, int slot, int j) {
      const uint32_t buf = lds_base + (uint32_t)(slot * kWideStepBytes);
      const int k0 = min(step, nsteps - 1) * 128;  // past the end: the last step again
      const int i = j >> 2, term = (j >> 1) & 1, rh = j & 1;
      const int plane = ((wave * 2 + i) * 2 + term) * 2 + rh;
      dma_load_16(cp_row[i][rh] + (size_t)term * Kp + k0, buf + (uint32_t)(plane * 1024));
    };
    // first byte of the 16 that hold group g's 12 (the last group starts early rather
    // than read past the row: see scale_index)
    auto row_scale_start = [&](int g) { return min(g * 12, sstride - 16); };
    auto weight_scale_start = [&](int g) { return min(g * 12, groups - 16); };
    auto copy_row_scales = [&](int g) {
      dma_load_16(cp_scale + row_scale_start(g),
                  lds_base + (uint32_t)(kWideRowScales + (g & 1) * 2048 + (wave & 1) * 1024));
    };
    // ---- weight copies: a tile's 64 x 16 bytes in lane order, per wavefront
    const uint32_t w_ring = lds_base + (uint32_t)(kWideWeights + wave * (R * 4096));
    const uint32_t ws_ring = lds_base + (uint32_t)(kWideWeightScales + wave * 2048);
    auto copy_weight_tile = [&](int step, int slot, int t) {  // past the end: the last group
      const int g = min(step * 4 + lq, groups - 1);
      dma_load_16(w_rows[t] + (size_t)g * 16, w_ring + (uint32_t)(slot * 4096 + t * 1024));
    };
    // lane (n, q) copies dword q of weight row n's 16 scale bytes: LDS [q][n] dwords
    auto copy_weight_scale_tile = [&](int g, int t) {
      const int b0 = weight_scale_start(g) + 4 * lq;
      dma_load_4(s_rows[t] + b0, ws_ring + (uint32_t)((g & 1) * 1024 + t * 256));
    };
    // operand reads of row tile m of a slot: lane (n, q) takes piece q (q + 4) of row n
    const int rd0 = (ln >> 3) * 1024 + (ln & 7) * 128 + ((lq ^ (ln & 7)) * 16);
    const int rd1 = rd0 ^ 64;
    auto read_rows = [&](int slot, int m, int step) {
      const uint8_t* tile = lds_bytes + slot * kWideStepBytes + m * 4096;
      Rows b;
      b.h0 = *reinterpret_cast<const u32x4*>(tile + rd0);
      b.h1 = *reinterpret_cast<const u32x4*>(tile + rd1);
      b.l0 = *reinterpret_cast<const u32x4*>(tile + 2048 + rd0);
      b.l1 = *reinterpret_cast<const u32x4*>(tile + 2048 + rd1);
      const int g = step / 3;  // uniform
      const int idx = step * 4 + lq - row_scale_start(g);
      b.sb = lds_bytes[kWideRowScales + (g & 1) * 2048 + (m * 16 + ln) * 16 + idx];
      return b;
    };

    f32x4 acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint32_t bad = 0u;

    // The K loop, compiled once per number of row tiles it multiplies (LIVE >= n_live:
    // straight-line code, so that the order reads of the next tile -> MFMAs of this
    // one survives; the tiles between n_live and LIVE are padding rows).
    auto k_loop = [&](auto live_c) {
      constexpr int LIVE = decltype(live_c)::value;
      // operation k (see above) of K step c, c % 3 = j
      auto issue = [&](int c, int j, int k) {
        if (k < 5) copy_row_piece(c + 2, (j + 2) % R, 3 + k);
        else if (k < 9) copy_weight_tile(c + R, j, k - 5);
        else if (k < 13) { if (j == 0) copy_weight_scale_tile(c / 3 + 1, k - 9); }
        else if (k < 16) copy_row_piece(c + R, j, k - 13);
        else if (j == 0) copy_row_scales(c / 3 + 1);
      };
      // The prologue issues what steps -3, -2, -1 would, less the row pieces of step -1.
#pragma unroll
      for (int j = 0; j < R; ++j) {
#pragma unroll
        for (int k = (j == 0 ? 5 : 0); k < 17; ++k) issue(j - R, j, k);
      }
      // all of steps 0's rows, weights and scale bytes have landed once only what was
      // issued after the late row pieces of step 0 is outstanding
      __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(kWeightOps + ops_after(1) + ops_before(2) + ops_after(2))
                       : "memory");
      __builtin_amdgcn_s_barrier();
      __asm__ volatile("" ::: "memory");
      Rows cur = read_rows(0, 0, 0);

      // MFMA operand and scale of weight tile t for K step cc from the weight ring
      // (lanes past K: the step's weights are the last group's again and meet zero
      // rows; their scale byte is made a neutral one).
      auto prep_tile = [&](int cc, int slot, int t, i32x8& wa, int& sa) {
        cc = min(cc, nsteps - 1);  // past the end the slot holds the last step again
        const uint8_t* wr = lds_bytes + kWideWeights + wave * (R * 4096) + slot * 4096 + t * 1024;
        const u32x4 w = *reinterpret_cast<const u32x4*>(wr + lane * 16);
        const int g = cc / 3;  // uniform
        const int idx = min(cc * 4 + lq, groups - 1) - weight_scale_start(g);
        uint32_t sbw = lds_bytes[kWideWeightScales + wave * 2048 + (g & 1) * 1024 + t * 256 +
                                 (idx >> 2) * 64 + ln * 4 + (idx & 3)];
        if (cc * 4 + lq >= groups) sbw = 127u;
        bad |= (uint32_t)((sbw - kScaleLo) > (kScaleHi - kScaleLo));
        bad |= fp4x8_nonfinite(w[0]) | fp4x8_nonfinite(w[1]) | fp4x8_nonfinite(w[2]) |
               fp4x8_nonfinite(w[3]);
        sa = (int)sbw - 1;
        wa = fp4_operand(w);
      };
      // operands of the current step in wa[c % 2], of the next in the other half
      i32x8 wa[2][NT];
      int sa[2][NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) prep_tile(0, 0, t, wa[0][t], sa[0][t]);

      // One row tile: its MFMAs in two halves (the leading terms, the remainders), a
      // memory operation ahead of each half, the vector work of the region (among it
      // the preparation of one of the next step's weight tiles) spread between the
      // MFMAs, during which the matrix pipe is busy anyway.
      auto tile = [&](int m, const i32x8 (&wa_)[NT], const int (&sa_)[NT], auto&& op_a, auto&& op_b) {
        // (opaque, so that no use of the byte moves up into the previous tile's
        // region and makes the MFMAs there wait for the read)
        int sbh = cur.sb;
        __asm__ volatile("" : "+v"(sbh));
        bad |= (uint32_t)(sbh == 0);
        const int sbl = sbh - 4;
        const i32x8 bh = fp8_operand(cur.h0, cur.h1);
        const i32x8 bl = fp8_operand(cur.l0, cur.l1);
        op_a();
        // the two MFMAs of an accumulator are kept NT instructions apart
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[m][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa_[t], bh, acc[m][t], 4, 0, 0,
                                                                       sa_[t], 0, sbh);
        __builtin_amdgcn_sched_barrier(0);
        op_b();
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[m][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa_[t], bl, acc[m][t], 4, 0, 0,
                                                                       sa_[t], 0, sbl);
        __builtin_amdgcn_sched_barrier(0);
      };

      // Two K steps per pass of the unrolled body would fix c % 2 but not c % 3; six do.
#pragma unroll 1
      for (int c0 = 0; c0 < nsteps; c0 += 2 * R) {
        auto step = [&](auto i_c) {
          constexpr int i = decltype(i_c)::value;
          constexpr int j = i % R, jn = (j + 1) % R, jp = (j + 2) % R, cb = i & 1, nb = cb ^ 1;
          // The unrolled body stops at the last step (uniform): a step's counted waits
          // look back at earlier operations only.
          const int c = c0 + i;
          if (c >= nsteps) return;
          const bool work = has_unit;  // uniform
          // The weights of step c + 1 (and, when that is a first step of three, their
          // scale bytes) were issued in step c - 2; since then: the early row pieces of
          // that step (and row scales) and all of step c - 1.
          constexpr int kWeightWait = ops_after(jn) + ops_before(jp) + ops_after(jp);
          __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(kWeightWait) : "memory");
          auto prep_next = [&](int t) { prep_tile(c + 1, jn, t, wa[nb][t], sa[nb][t]); };
          // operations before the barrier: two per row tile but the last (all at once
          // where the step has a single tile, or does no arithmetic)
          constexpr int kBefore = 13;
          constexpr int kSlots = LIVE > 1 ? 2 * (LIVE - 1) : 1;  // places between the tiles' halves
          constexpr int kPer = (kBefore + kSlots - 1) / kSlots;
          auto before = [&](int first) {
#pragma unroll
            for (int k = first; k < first + kPer; ++k)
              if (k < kBefore) issue(c, j, k);
          };
          if (work && LIVE > 1) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m + 1 < LIVE; ++m) {
              const Rows nxt = read_rows(j, m + 1, c);
              if (m < NT) prep_next(m);
              tile(m, wa[cb], sa[cb], [&]() { before(2 * m * kPer); }, [&]() { before((2 * m + 1) * kPer); });
              cur = nxt;
            }
          } else {
#pragma unroll
            for (int k = 0; k < kBefore; ++k) issue(c, j, k);
          }
          // Before the last tile: this wavefront's row copies of step c + 1 (the early
          // pieces, with the row scales if c + 1 is a first step of three, from after
          // the barrier of step c - 2; the late ones from step c - 1) have landed and
          // its reads of step c are complete; after the barrier that holds for every
          // wavefront, so slot j takes the early pieces of step c + 3 and step c + 1
          // can be read.  Outstanding may be what followed the late pieces in step
          // c - 1 and what this step has issued so far.
          constexpr int kRowWait = kWeightOps + (jp == 0 ? NT : 0) + ops_after(jp) + ops_before(j);
          __asm__ volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kRowWait) : "memory");
          __builtin_amdgcn_s_barrier();
          __asm__ volatile("" ::: "memory");
          if (work) {
            __builtin_amdgcn_sched_barrier(0);
            const Rows nxt = read_rows(jn, 0, c + 1);
#pragma unroll
            for (int t = LIVE - 1; t < NT; ++t) prep_next(t);
            tile(LIVE - 1, wa[cb], sa[cb], [&]() { issue(c, j, 13); issue(c, j, 14); },
                 [&]() { issue(c, j, 15); issue(c, j, 16); });
            cur = nxt;
          } else {
#pragma unroll
            for (int k = 13; k < 17; ++k) issue(c, j, k);
          }
        };
        step(IntC<0>{});
        step(IntC<1>{});
        step(IntC<2>{});
        step(IntC<3>{});
        step(IntC<4>{});
        step(IntC<5>{});
      }
    };
    if (n_live > 6) k_loop(IntC<8>{});
    else if (n_live > 4) k_loop(IntC<6>{});
    else if (n_live > 2) k_loop(IntC<4>{});
    else if (n_live == 2) k_loop(IntC<2>{});
    else k_loop(IntC<1>{});
    // the copies past the last step land in the ring, which the epilogue reuses
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __syncthreads();

    // Stage 0: the zero blocks and scale bytes between ncols and the next multiple of
    // 128 of the act split rows, written by the workgroups of the first columns.
    if (STAGE == 0 && p.actq != nullptr && blockIdx.x == 0 && tid < n_rows && row_flat[tid] >= 0) {
      const int ip = split_row_k(p.ncols);
      uint8_t* qrow = p.actq + (size_t)(row0 + tid) * (size_t)ip * 2;
      for (int k = p.ncols; k < ip; k += 16) {
        *reinterpret_cast<u32x4*>(qrow + k) = u32x4{0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4*>(qrow + ip + k) = u32x4{0u, 0u, 0u, 0u};
      }
      uint8_t* srow_s = p.actqs + (size_t)(row0 + tid) * (size_t)split_scale_stride(p.ncols);
      for (int g = p.ncols / 32; g < ip / 32; ++g) srow_s[g] = 127u;
    }
    if (STAGE == 1 && p.pos != nullptr && blockIdx.x == 0 && tid < n_rows && row_flat[tid] >= 0)
      p.pos[row_flat[tid]] = row0 + tid;
    if (!has_unit) return;

    // ---- epilogue; the exact path where the fast one was outside its domain -------
    // (a scale byte 0 among a column's blocks marks rows outside the range: the
    // whole unit is redone, from the bf16 rows)
    const bool redo = __ballot(bad != 0u) != 0ull;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m >= n_live) break;
      const int flat = row_flat[m * 16 + ln];
      const int srow = row0 + m * 16 + ln;
      if (redo) {
        const uint16_t* a_row = nullptr;
        if (flat >= 0) a_row = p.A + (size_t)(STAGE == 0 ? flat / p.top_k : srow) * (size_t)p.a_stride;
        exact_unit_global<NT>(w_rows, s_rows, a_row, K, lane, acc[m]);
      }
      if (STAGE == 0) {
        uint2 packed[NT / 2] = {};
        if (flat >= 0) epilogue_tile<STAGE, NT>(p, e, acc[m], col0, flat, srow, lq, packed);
        if (p.actq != nullptr)
          store_split_act(p, col0[0], col0[1], flat, srow, lane, packed[0], packed[1]);
      } else if (p.y != nullptr) {
        // plain stores of the row's 4 x 4 columns; combine_kernel sums the tokens' rows
        if (flat >= 0) {
          const float w = p.topk_w[flat];
          float* yrow = p.y + (size_t)srow * (size_t)p.ncols;
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            const int c = col0[t] + 4 * lq;
            f32x4 v = acc[m][t];
            if (p.bias != nullptr)
              v += *reinterpret_cast<const f32x4u*>(p.bias + (size_t)e * (size_t)p.ncols + c);
            *reinterpret_cast<f32x4*>(yrow + c) = v * w;
          }
        }
      } else {
        // Transposed through this wavefront's part of the (now idle) ring, so
        // that one atomic instruction adds 64 consecutive columns of one token
        // instead of 4 x 4 scattered columns of 16 tokens.
        constexpr int kRowStride = 16 * NT + 4;  // floats; the pad spreads the rows over the banks
        float* tr = reinterpret_cast<float*>(wide_lds) + (size_t)wave * 16 * kRowStride;
#pragma unroll
        for (int t = 0; t < NT; ++t)
          *reinterpret_cast<f32x4*>(tr + ln * kRowStride + t * 16 + 4 * lq) = acc[m][t];
        const int c = col0[0] + lane;  // the unit's 16 NT columns are consecutive
        const float b = p.bias != nullptr ? p.bias[(size_t)e * (size_t)p.ncols + c] : 0.0f;
#pragma unroll 4
        for (int i = 0; i < 16; ++i) {
          const int fi = row_flat[m * 16 + i];  // uniform
          if (fi < 0) continue;
          const float v = tr[i * kRowStride + lane];
          unsafeAtomicAdd(p.out + (size_t)(fi / p.top_k) * (size_t)p.ncols + c, (v + b) * p.topk_w[fi]);
        }
      }
    }
  };

  const int total_rows = p.num_blocks * p.block_size;
  const int win = wide_window_rows(p.block_size);
  int row = blockIdx.y * win;
  const int win_end = min(row + win, total_rows);
  while (row < win_end) {  // uniform
    const int e = p.expert_ids[row / p.block_size];
    int seg_end = min(win_end, (row / p.block_size + 1) * p.block_size);
    while (seg_end < win_end && p.expert_ids[seg_end / p.block_size] == e)
      seg_end = min(win_end, seg_end + p.block_size);
    if (e >= 0) segment(row, seg_end - row, e);
    row = seg_end;
  }
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* dst, int32_t value, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

// out[t, :] (+)= the sum over the token's selections s, in order, of y[pos[t * top_k + s], :]
// (selections whose expert is not local have pos < 0).  One thread per 4 columns.  TOPK > 0:
// top_k known at compile time, so that a thread asks for all of a token's rows before it
// adds the first (one load in flight per thread leaves a quarter of the bandwidth unused);
// a selection that is not local adds zeros, which changes no bit of a sum that starts at +0.
template <int TOPK>
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ y,
                                                      const int32_t* __restrict__ pos,
                                                      float* __restrict__ out, int M, int top_k,
                                                      int ncols, int overwrite) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= ncols) return;
  for (int t = blockIdx.y; t < M; t += gridDim.y) {  // grid.y is capped at 65535
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if constexpr (TOPK > 0) {
      int r[TOPK];
      f32x4 v[TOPK];
#pragma unroll
      for (int s = 0; s < TOPK; ++s) r[s] = pos[t * TOPK + s];  // uniform
#pragma unroll
      for (int s = 0; s < TOPK; ++s) {
        v[s] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (r[s] >= 0) v[s] = *reinterpret_cast<const f32x4*>(y + (size_t)r[s] * (size_t)ncols + c);
      }
#pragma unroll
      for (int s = 0; s < TOPK; ++s) sum += v[s];
    } else {
      for (int s = 0; s < top_k; ++s) {
        const int r = pos[t * top_k + s];  // uniform
        if (r >= 0) sum += *reinterpret_cast<const f32x4*>(y + (size_t)r * (size_t)ncols + c);
      }
    }
    f32x4* o = reinterpret_cast<f32x4*>(out + (size_t)t * (size_t)ncols + c);
    *o = overwrite ? sum : *o + sum;
  }
}

// bf16 rows [R, K] -> split rows (see GemmArgs::Aq), zero blocks between K and
// split_row_k(K) included.  One lane per 8 values; the four lanes of a block of 32
// are a quad (K is a multiple of 32, so no block straddles two rows or the end of K).
__global__ __launch_bounds__(256) void split_rows_kernel(const uint16_t* __restrict__ x,
                                                         uint8_t* __restrict__ xq,
                                                         uint8_t* __restrict__ xs, long long pieces,
                                                         int K) {
  const int kp = split_row_k(K);
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // piece index, 8 values
  const long long row = i / (kp / 8);
  const int k = (int)(i - row * (kp / 8)) * 8;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (i < pieces && k < K) v = *reinterpret_cast<const u32x4*>(x + row * K + k);
  uint32_t emax = bf16x8_max_exponent(v);
  emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0xB1, 0xF, 0xF, true));
  emax = max(emax, (uint32_t)__builtin_amdgcn_mov_dpp((int)emax, 0x4E, 0xF, 0xF, true));
  uint32_t sb = emax - 7u, stored;
  if (emax == 0u) sb = 127u;
  stored = sb;
  if (emax != 0u && (sb < kScaleLo || sb > kScaleHi)) { stored = 0u; sb = 127u; }
  uint2 hi, lo;
  split_bf16x8(v, sb, hi, lo);
  if (i < pieces) {
    uint8_t* qrow = xq + row * 2 * kp;
    *reinterpret_cast<uint2*>(qrow + k) = hi;
    *reinterpret_cast<uint2*>(qrow + kp + k) = lo;
    if ((k & 31) == 0) xs[row * split_scale_stride(K) + (k >> 5)] = (uint8_t)stored;
  }
}

int num_compute_units() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return 256;
    return n;
  }();
  return cus;
}

constexpr size_t kResidentLdsLimit = 150 * 1024;  // dynamic LDS the resident kernel may ask for
// ... and its routed forms, whose tables are 14 KB of static LDS over the plain form's
constexpr size_t kRoutedStaticLds = 14 * 1024;
constexpr size_t kRoutedLdsLimit = kResidentLdsLimit - kRoutedStaticLds;

// True when the device grants the kernel its dynamic LDS (asked once per kernel;
// a refusal makes the caller take the other variant).
template <int STAGE, int WAVES, int NT, int D, bool KSPLIT = false, int ROUTE = 0, bool PACKED = false,
          bool WIDEK = false>
bool resident_kernel_ready() {
  static const bool configured = [] {
    const hipError_t err = hipFuncSetAttribute(
        reinterpret_cast<const void*>(stream_resident_kernel<STAGE, WAVES, NT, D, KSPLIT, ROUTE, PACKED, WIDEK>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(ROUTE != 0 ? kRoutedLdsLimit : kResidentLdsLimit));
    if (err != hipSuccess) (void)hipGetLastError();  // not left for the next caller to find
    return err == hipSuccess;
  }();
  return configured;
}

template <int STAGE, int WAVES, int NT, int D, bool KSPLIT = false, int ROUTE = 0, bool PACKED = false,
          bool WIDEK = false>
bool launch_resident(const GemmArgs& g, size_t lds, hipStream_t stream) {
  if (!resident_kernel_ready<STAGE, WAVES, NT, D, KSPLIT, ROUTE, PACKED, WIDEK>()) return false;
  hipLaunchKernelGGL((stream_resident_kernel<STAGE, WAVES, NT, D, KSPLIT, ROUTE, PACKED, WIDEK>), dim3(num_compute_units()),
                     dim3(64 * WAVES), lds, stream, g);
  return true;
}

template <int STAGE, int NT, int D, int MT, bool ONE = false>
bool chunked_kernel_ready() {
  static const bool configured = [] {
    const hipError_t err = hipFuncSetAttribute(
        reinterpret_cast<const void*>(stream_chunked_kernel<STAGE, NT, D, MT, ONE>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)chunked_lds_bytes(MT));
    if (err != hipSuccess) (void)hipGetLastError();  // not left for the next caller to find
    return err == hipSuccess;
  }();
  return configured;
}

template <int STAGE, int NT, int D, int MT, bool ONE = false>
bool launch_chunked(const GemmArgs& g, size_t lds, hipStream_t stream) {
  if (!chunked_kernel_ready<STAGE, NT, D, MT, ONE>()) return false;
  hipLaunchKernelGGL((stream_chunked_kernel<STAGE, NT, D, MT, ONE>), dim3(num_compute_units()),
                     dim3(64 * kChunkWaves), lds, stream, g);
  return true;
}

// The chunked kernel's single-chunk form: the second stage's, for rows of up to 2048 values.
template <int STAGE>
bool chunked_one_applies(const GemmArgs& g) {
  return STAGE == 1 && (g.K / 32 + 3) / 4 <= 2 * kChunkSteps;
}

// Launch shape of one stage.  variant kMoeVariantLds = the tile kernel.
struct StagePlan {
  int variant, waves, nt, depth;
  bool ksplit;  // the resident kernel with K shared between the wavefronts of a unit
  bool packed;  // ... reading the prepacked form (whenever the caller gives it)
  bool widek;   // ... its instantiation for rows of 3072 < K <= 4096 with 8 wavefronts
  bool chunked; // the chunked decode kernel (prepacked form), `mt` 16-row tiles a pass
  int mt;
  size_t resident_lds;
};

template <int STAGE>
StagePlan plan_stage(const GemmArgs& g) {
  // a record of the tuning store first, then the compiled-in rules
  MoeTile tile;
  // The prepacked form whenever the caller gives it: its decode kernels are the faster
  // ones (no scale block to park, nothing to check or fix in the loop).
  const bool packed = g.Wp != nullptr && !(STAGE == 0 && g.ncols % 64 != 0);
  if (!moe_tuning_find(STAGE, g.K, g.ncols, g.n_flat, &tile))
    tile = pick_moe_tile(g.n_flat, g.K, g.ncols, STAGE, packed,
                         packed && (g.block_size == 16 || g.block_size == 32) ? g.p_experts : 0, g.block_size);
  StagePlan pl;
  pl.packed = packed;
  pl.chunked = false;
  pl.mt = 1;
  if (tile.variant == kMoeVariantChunked) {  // one of the decode kernels for the callers
    pl.chunked = true;
    pl.mt = g.block_size / 16;
    pl.variant = kMoeVariantResident;
    pl.ksplit = false;
    pl.widek = false;
    pl.nt = tile.nt;
    pl.depth = tile.depth;
    pl.waves = tile.waves;
    pl.resident_lds = chunked_lds_bytes(pl.mt);
    const int c_units = STAGE == 0 ? g.ncols / (8 * pl.nt) : g.ncols / (16 * pl.nt);
    if (!packed || (g.block_size != 16 && g.block_size != 32) || g.num_blocks > kMaxRuns ||
        g.ncols % 16 != 0 || c_units < 1 || pl.waves != kChunkWaves)
      pl.variant = kMoeVariantLds;
    return pl;
  }
  pl.ksplit = tile.variant == kMoeVariantResidentKSplit;
  pl.variant = pl.ksplit ? (int)kMoeVariantResident : tile.variant;
  pl.nt = tile.nt;
  pl.depth = tile.depth;
  pl.waves = tile.waves;
  const int groups = g.K / 32;
  const int nsteps = (groups + 3) / 4;
  // operand planes + block scales + one weight-scale region per wavefront
  pl.resident_lds = (size_t)nsteps * (4096 + 64) + (packed ? 0 : (size_t)pl.waves * pl.nt * 16 * groups);
  // (K split: the partial sums of the wavefronts, 1 KB a tile, lie over the operand planes)
  if (pl.ksplit && (size_t)nsteps * 4096 < (size_t)pl.waves * pl.nt * 1024) pl.ksplit = false;
  const int res_units = STAGE == 0 ? g.ncols / (8 * pl.nt) : g.ncols / (16 * pl.nt);
  // (the wide instantiations exist for the two shapes the rules return at such K)
  pl.widek = packed && STAGE == 0 && pl.waves == 8 && nsteps * 4 > resident_batch(8) * 8 && pl.nt == 2 &&
             (pl.ksplit ? pl.depth == 4 : pl.depth == 2);
  if (pl.resident_lds > kResidentLdsLimit || g.num_blocks > kMaxRuns ||
      (!packed && pl.nt * groups > 64 * resident_scale_pieces(pl.waves)) ||
      (res_units + pl.waves - 1) / pl.waves > 64 ||  // one bit per unit in a wavefront's redo mask
      nsteps * 4 > resident_batch(pl.waves, pl.widek) * pl.waves)  // the rows are staged in one batch
    pl.variant = kMoeVariantLds;
  return pl;
}

// True when the device grants the wide kernel its LDS (asked once per stage).
template <int STAGE>
bool wide_kernel_ready() {
  static const bool configured = [] {
    const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(tile_wide_kernel<STAGE>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               kWideLdsBytes);
    if (err != hipSuccess) (void)hipGetLastError();  // not left for the next caller to find
    return err == hipSuccess;
  }();
  return configured;
}

// The wide kernel takes split rows (launch_fused_moe sets Aq only where it applies: a
// tile-kernel stage with K >= 512, whose scale bytes it reads sixteen at a time, on a
// device that grants its LDS).
bool wide_kernel_applies(const GemmArgs& g) { return g.Aq != nullptr; }

template <int STAGE>
void launch_stage(const GemmArgs& g, const StagePlan& pl, hipStream_t stream) {
  // (a stage without raw weights that is not resident is kept away from here by the callers)
  if (pl.variant == kMoeVariantResident && pl.chunked) {
#define VK_CHUNKED(S_, W_, NT_, D_) \
  if constexpr (STAGE == S_) { \
    if (pl.nt == NT_ && pl.depth == D_) { \
      if constexpr (S_ == 1) { \
        if (chunked_one_applies<S_>(g) && \
            (pl.mt == 2 ? launch_chunked<S_, NT_, D_, 2, true>(g, pl.resident_lds, stream) \
                        : launch_chunked<S_, NT_, D_, 1, true>(g, pl.resident_lds, stream))) \
          return; \
      } \
      if (pl.mt == 2 ? launch_chunked<S_, NT_, D_, 2>(g, pl.resident_lds, stream) \
                     : launch_chunked<S_, NT_, D_, 1>(g, pl.resident_lds, stream)) \
        return; \
    } \
  }
    VK_CHUNKED_VARIANTS(VK_CHUNKED)
#undef VK_CHUNKED
    return;
  }
  if (pl.packed && pl.variant == kMoeVariantResident && pl.widek) {
    if constexpr (STAGE == 0) {
      if (pl.ksplit) (void)launch_resident<0, 8, 2, 4, true, 0, true, true>(g, pl.resident_lds, stream);
      else (void)launch_resident<0, 8, 2, 2, false, 0, true, true>(g, pl.resident_lds, stream);
    }
    return;
  }
  if (pl.packed && pl.variant == kMoeVariantResident) {
#define VK_RESIDENT(S_, W_, NT_, D_) \
  if constexpr (STAGE == S_) { \
    if (pl.ksplit && pl.waves == W_ && pl.nt == NT_ && pl.depth == D_ && \
        launch_resident<S_, W_, NT_, D_, true, 0, true>(g, pl.resident_lds, stream)) \
      return; \
  }
    VK_KSPLIT_VARIANTS(VK_RESIDENT)
#undef VK_RESIDENT
#define VK_RESIDENT(S_, W_, NT_, D_) \
  if constexpr (STAGE == S_) { \
    if (pl.waves == W_ && pl.nt == NT_ && pl.depth == D_ && \
        launch_resident<S_, W_, NT_, D_, false, 0, true>(g, pl.resident_lds, stream)) \
      return; \
  }
    VK_RESIDENT_VARIANTS(VK_RESIDENT)
#undef VK_RESIDENT
    return;
  }
  if (pl.variant == kMoeVariantResident) {
#define VK_RESIDENT(S_, W_, NT_, D_) \
  if constexpr (STAGE == S_) { \
    if (pl.ksplit && pl.waves == W_ && pl.nt == NT_ && pl.depth == D_ && \
        launch_resident<S_, W_, NT_, D_, true>(g, pl.resident_lds, stream)) \
      return; \
  }
    VK_KSPLIT_VARIANTS(VK_RESIDENT)
#undef VK_RESIDENT
#define VK_RESIDENT(S_, W_, NT_, D_) \
  if constexpr (STAGE == S_) { \
    if (pl.waves == W_ && pl.nt == NT_ && pl.depth == D_ && \
        launch_resident<S_, W_, NT_, D_>(g, pl.resident_lds, stream)) \
      return; \
  }
    VK_RESIDENT_VARIANTS(VK_RESIDENT)
#undef VK_RESIDENT
  }
  const int units = STAGE == 0 ? g.ncols / (8 * kTileNT) : g.ncols / (16 * kTileNT);
  const int group_rows = tile_group_rows(g.block_size, 16 * kTileMT);
  const dim3 grid((units + kTileWaves - 1) / kTileWaves, g.num_blocks * (g.block_size / group_rows));
  if (wide_kernel_applies(g)) {
    const int wide_units = STAGE == 0 ? g.ncols / (8 * kWideNT) : g.ncols / (16 * kWideNT);
    const int win = wide_window_rows(g.block_size);
    const dim3 grid_wide((wide_units + kWideWaves - 1) / kWideWaves,
                         (g.num_blocks * g.block_size + win - 1) / win);
    hipLaunchKernelGGL((tile_wide_kernel<STAGE>), grid_wide, dim3(64 * kWideWaves), kWideLdsBytes,
                       stream, g);
    return;
  }
  hipLaunchKernelGGL((tile_gemm_kernel<STAGE>), grid, dim3(64 * kTileWaves), 0, stream, g);
}

// Workspace of the fused call: split rows of A, then of act, each followed by
// its scale bytes; then the second stage's rows before the combine (fp32,
// [EM, hidden]) and the sorted position of every flat index.
struct Workspace {
  uint8_t* a_q;
  uint8_t* a_s;
  uint8_t* act_q;
  uint8_t* act_s;
  float* y;
  int32_t* pos;
};

struct WorkspaceLayout {
  size_t aq, as, cq, cs, y, pos;
  size_t total() const { return aq + as + cq + cs + y + pos; }
};

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

WorkspaceLayout workspace_layout(int M, int hidden, int ispp, int top_k, int EM) {
  WorkspaceLayout l;
  l.aq = align256((size_t)M * split_row_k(hidden) * 2);
  l.as = align256((size_t)M * split_scale_stride(hidden));
  l.cq = align256((size_t)EM * split_row_k(ispp) * 2);
  l.cs = align256((size_t)EM * split_scale_stride(ispp));
  l.y = align256((size_t)EM * hidden * sizeof(float));
  l.pos = align256((size_t)M * top_k * sizeof(int32_t));
  return l;
}

bool carve_workspace(const FusedMoeArgs& a, Workspace& w) {
  if (a.workspace == nullptr) return false;
  const WorkspaceLayout l = workspace_layout(a.M, a.hidden, a.ispp, a.top_k, a.EM);
  if (a.workspace_bytes < l.total()) return false;
  uint8_t* base = static_cast<uint8_t*>(a.workspace);
  if ((reinterpret_cast<uintptr_t>(base) & 15) != 0) return false;
  w.a_q = base;
  w.a_s = w.a_q + l.aq;
  w.act_q = w.a_s + l.as;
  w.act_s = w.act_q + l.cq;
  w.y = reinterpret_cast<float*>(w.act_s + l.cs);
  w.pos = reinterpret_cast<int32_t*>(w.act_s + l.cs + l.y);
  return true;
}

GemmArgs common_args(const FusedMoeArgs& a) {
  GemmArgs g{};
  g.sorted_ids = a.sorted_ids;
  g.expert_ids = a.expert_ids;
  g.topk_w = a.topk_w;
  g.act = a.act;
  g.out = a.out;
  g.n_flat = a.M * a.top_k;
  g.top_k = a.top_k;
  g.num_blocks = a.EM / a.block_size;
  g.block_size = a.block_size;
  g.swiglu_limit = a.swiglu_limit;
  g.beta = a.beta;
  g.linear_beta = a.linear_beta;
  g.activation = a.activation;
  return g;
}

GemmArgs gateup_args(const FusedMoeArgs& a) {
  GemmArgs g = common_args(a);
  g.A = a.A;
  g.W = a.w13;
  g.Ws = a.w13_scale;
  if (a.w13_packed != nullptr) {
    g.p_units = mx_units(0, a.ispp);
    g.p_experts = a.num_experts;
    g.Wp = a.w13_packed;
    g.Wpf = a.w13_packed + mx_packed_body_bytes(a.num_experts, g.p_units, mx_kp(a.hidden) / 128);
  }
  g.bias = a.b13;
  g.K = a.hidden;
  g.a_stride = a.hidden;
  g.ncols = a.ispp;
  return g;
}

GemmArgs down_args(const FusedMoeArgs& a) {
  GemmArgs g = common_args(a);
  g.A = a.act;
  g.W = a.w2;
  g.Ws = a.w2_scale;
  if (a.w2_packed != nullptr) {
    g.p_units = mx_units(1, a.hidden);
    g.p_experts = a.num_experts;
    g.Wp = a.w2_packed;
    g.Wpf = a.w2_packed + mx_packed_body_bytes(a.num_experts, g.p_units, mx_kp(a.ispp) / 128);
  }
  g.bias = a.b2;
  g.K = a.ispp;
  g.a_stride = a.ispp;
  g.ncols = a.hidden;
  return g;
}

}  // namespace

// A call that passes the prepacked weights alone (w13 / w2 null): true when the library
// can run it -- both stages on the decode kernels' packed forms, or the workspace the
// prepacked kernels need.
bool fused_moe_packed_only_ok(const FusedMoeArgs& a) {
  if (a.w13_packed == nullptr || a.w2_packed == nullptr || a.num_experts <= 0) return false;
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return true;  // nothing will run
  const GemmArgs g0 = gateup_args(a), g1 = down_args(a);
  const StagePlan p0 = plan_stage<0>(g0), p1 = plan_stage<1>(g1);
  if (p0.variant == kMoeVariantResident && p1.variant == kMoeVariantResident && p0.packed && p1.packed) return true;
  return fused_moe_prepacked_takes(a, true);
}

bool moe_gateup_packed_only_ok(const FusedMoeArgs& a) {
  if (a.w13_packed == nullptr || a.num_experts <= 0) return false;
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return true;
  const GemmArgs g = gateup_args(a);
  const StagePlan pl = plan_stage<0>(g);
  return pl.packed && pl.variant == kMoeVariantResident;
}

bool moe_down_packed_only_ok(const FusedMoeArgs& a) {
  if (a.w2_packed == nullptr || a.num_experts <= 0) return false;
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return true;
  const GemmArgs g = down_args(a);
  const StagePlan pl = plan_stage<1>(g);
  if (pl.variant == kMoeVariantResident && pl.packed) return true;
  return fused_moe_prepacked_takes(a, false);
}

size_t fused_moe_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM) {
  if (M <= 0 || EM <= 0 || hidden <= 0 || ispp <= 0 || top_k <= 0) return 0;
  // enough for either layout (raw weights, prepacked weights)
  const size_t raw = workspace_layout(M, hidden, ispp, top_k, EM).total();
  const size_t packed = mx_workspace_bytes(M, hidden, ispp, top_k, EM);
  return raw > packed ? raw : packed;
}

void launch_fill_i32(int32_t* dst, int32_t value, int n, hipStream_t stream) {
  if (n <= 0) return;
  hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, dst,
                     value, n);
}

void launch_combine(const float* y, const int32_t* pos, float* out, int M, int top_k, int hidden,
                    bool overwrite, hipStream_t stream) {
  const dim3 grid((unsigned)((hidden / 4 + 255) / 256), (unsigned)(M < 65535 ? M : 65535));
  const int ow = overwrite ? 1 : 0;
  switch (top_k) {
#define VK_COMBINE(K_)                                                                              \
  case K_:                                                                                          \
    hipLaunchKernelGGL(combine_kernel<K_>, grid, dim3(256), 0, stream, y, pos, out, M, top_k, hidden, ow); \
    break;
    VK_COMBINE(2) VK_COMBINE(4) VK_COMBINE(6) VK_COMBINE(8)
#undef VK_COMBINE
    default:
      hipLaunchKernelGGL(combine_kernel<0>, grid, dim3(256), 0, stream, y, pos, out, M, top_k, hidden, ow);
  }
}

bool prepare_moe_kernels() {
  bool ok = wide_kernel_ready<0>() && wide_kernel_ready<1>() && prepare_mx_kernels();
#define VK_READY(S_, W_, NT_, D_) ok = resident_kernel_ready<S_, W_, NT_, D_>() && ok;
  VK_RESIDENT_VARIANTS(VK_READY)
#undef VK_READY
#define VK_READY(S_, W_, NT_, D_) ok = resident_kernel_ready<S_, W_, NT_, D_, true>() && ok;
  VK_KSPLIT_VARIANTS(VK_READY)
#undef VK_READY
  ok = resident_kernel_ready<0, 8, 2, 4, true, 1>() && resident_kernel_ready<0, 8, 2, 2, false, 1>() && ok;
  ok = resident_kernel_ready<0, 4, 2, 8, false, 1>() && resident_kernel_ready<0, 4, 2, 8, false, 1, true>() && ok;
  ok = resident_kernel_ready<0, 8, 2, 2, false, 0, true, true>() && resident_kernel_ready<0, 8, 2, 4, true, 0, true, true>() && ok;
  ok = resident_kernel_ready<0, 8, 2, 2, false, 1, true, true>() && resident_kernel_ready<0, 8, 2, 4, true, 1, true, true>() && ok;
  ok = resident_kernel_ready<0, 8, 2, 2, false, 2, true, true>() && ok;
  ok = resident_kernel_ready<0, 8, 2, 2, false, 2>() && resident_kernel_ready<0, 4, 2, 8, false, 2>() && ok;
#define VK_READY(S_, W_, NT_, D_) ok = resident_kernel_ready<S_, W_, NT_, D_, false, 0, true>() && ok;
  VK_RESIDENT_VARIANTS(VK_READY)
#undef VK_READY
#define VK_READY(S_, W_, NT_, D_) ok = resident_kernel_ready<S_, W_, NT_, D_, true, 0, true>() && ok;
  VK_KSPLIT_VARIANTS(VK_READY)
#undef VK_READY
  ok = resident_kernel_ready<0, 8, 2, 4, true, 1, true>() && resident_kernel_ready<0, 8, 2, 2, false, 1, true>() && ok;
  ok = resident_kernel_ready<0, 8, 2, 2, false, 2, true>() && resident_kernel_ready<0, 4, 2, 8, false, 2, true>() && ok;
#define VK_READY(S_, W_, NT_, D_) \
  ok = chunked_kernel_ready<S_, NT_, D_, 1>() && chunked_kernel_ready<S_, NT_, D_, 2>() && ok; \
  if constexpr (S_ == 1) \
    ok = chunked_kernel_ready<S_, NT_, D_, 1, true>() && chunked_kernel_ready<S_, NT_, D_, 2, true>() && ok;
  VK_CHUNKED_VARIANTS(VK_READY)
#undef VK_READY
  MoeTile unused;
  (void)moe_tuning_find(0, 64, 64, 1, &unused);  // reads the tuning store now rather than on the first launch
  return ok;
}

// Router, alignment and the layer with the alignment inside the first stage's decode
// kernel (its routed forms), whose workgroup 0 writes the tables out for the second stage
// and the caller.  Up to kRouteMaxTokens tokens the kernel routes as well: two launches a
// step.  Beyond, up to kRouteMaxRows routed rows, the router has its launch and the kernel
// aligns from its ids: three launches instead of four, and no run listing in the kernel.
// False (nothing enqueued) when the call is not one these forms take: more routed rows or
// more than kRouteMaxExperts experts, a block size other than 16, a first stage whose
// launch shape has no routed form, or LDS that does not hold the tables as well.
bool launch_routed_moe(const FusedMoeArgs& a, const RoutedArgs& r, hipStream_t stream) {
  if (a.M <= 0 || a.M * a.top_k > kRouteMaxRows || r.num_experts > kRouteMaxExperts ||
      r.num_experts <= 0 || a.top_k > r.num_experts || a.block_size != 16 ||
      r.max_EM < 16 || r.max_EM % 16 != 0 || r.max_EM / 16 > kMaxRuns)
    return false;
  const bool route_inside = a.M <= kRouteMaxTokens && a.top_k <= 64;
  FusedMoeArgs b = a;
  b.EM = r.max_EM;
  GemmArgs g0 = gateup_args(b);
  GemmArgs g1 = down_args(b);
  const StagePlan p0 = plan_stage<0>(g0), p1 = plan_stage<1>(g1);
  if (p0.variant != kMoeVariantResident || p1.variant != kMoeVariantResident) return false;
  if (p0.chunked) return false;              // (the chunked kernel has no routed form)
  if (p0.packed != p1.packed) return false;  // (both packed forms or neither)
  if (p0.resident_lds > kRoutedLdsLimit) return false;
  g0.rt_logits = r.logits;
  g0.rt_expert_map = r.expert_map;
  g0.rt_topk_ids = r.topk_ids;
  g0.rt_topk_w = r.topk_w;
  g0.rt_sorted_ids = r.sorted_ids;
  g0.rt_expert_ids = r.expert_ids;
  g0.rt_out_em = r.out_EM;
  g0.rt_experts = r.num_experts;
  g0.rt_local_n = r.local_n;
  g0.rt_renormalize = r.renormalize;
  g0.rt_max_em = r.max_EM;
  g0.sorted_ids = nullptr;
  g0.expert_ids = nullptr;
  const bool overwrite = (a.flags & 1u) != 0u;  // VK_HIP_MOE_OVERWRITE_OUT
  if (overwrite) {
    g0.zero_out = a.out;
    g0.zero_count = (long long)a.M * a.hidden;
  }
  // the routed instantiation of the planned shape: is it there and ready?
  const int shape = p0.ksplit && p0.waves == 8 && p0.nt == 2 && p0.depth == 4 ? 1
                    : !p0.ksplit && p0.waves == 8 && p0.nt == 2 && p0.depth == 2 ? 2
                    : !p0.ksplit && p0.waves == 4 && p0.nt == 2 && p0.depth == 8 ? 3
                    : 0;
  bool ready = false;
  if (p0.widek) {  // (shape 1 or 2, prepacked form)
    if (route_inside) ready = shape == 1 ? resident_kernel_ready<0, 8, 2, 4, true, 1, true, true>()
                                         : resident_kernel_ready<0, 8, 2, 2, false, 1, true, true>();
    else ready = shape == 2 && resident_kernel_ready<0, 8, 2, 2, false, 2, true, true>();
    if (!ready) return false;
    if (route_inside) {
      if (shape == 1) launch_resident<0, 8, 2, 4, true, 1, true, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 8, 2, 2, false, 1, true, true>(g0, p0.resident_lds, stream);
    } else {
      launch_route_topk(r.logits, a.M, r.num_experts, a.top_k, r.renormalize, r.topk_ids, r.topk_w, stream);
      launch_resident<0, 8, 2, 2, false, 2, true, true>(g0, p0.resident_lds, stream);
    }
    g1.topk_w = r.topk_w;
    launch_stage<1>(g1, p1, stream);
    return true;
  }
  if (route_inside) {
    if (shape == 1) ready = p0.packed ? resident_kernel_ready<0, 8, 2, 4, true, 1, true>() : resident_kernel_ready<0, 8, 2, 4, true, 1>();
    if (shape == 2) ready = p0.packed ? resident_kernel_ready<0, 8, 2, 2, false, 1, true>() : resident_kernel_ready<0, 8, 2, 2, false, 1>();
    if (shape == 3) ready = p0.packed ? resident_kernel_ready<0, 4, 2, 8, false, 1, true>() : resident_kernel_ready<0, 4, 2, 8, false, 1>();
  } else {
    if (shape == 2) ready = p0.packed ? resident_kernel_ready<0, 8, 2, 2, false, 2, true>() : resident_kernel_ready<0, 8, 2, 2, false, 2>();
    if (shape == 3) ready = p0.packed ? resident_kernel_ready<0, 4, 2, 8, false, 2, true>() : resident_kernel_ready<0, 4, 2, 8, false, 2>();
  }
  if (!ready) return false;
  if (route_inside) {
    if (shape == 1) {
      if (p0.packed) launch_resident<0, 8, 2, 4, true, 1, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 8, 2, 4, true, 1>(g0, p0.resident_lds, stream);
    } else if (shape == 3) {
      if (p0.packed) launch_resident<0, 4, 2, 8, false, 1, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 4, 2, 8, false, 1>(g0, p0.resident_lds, stream);
    } else {
      if (p0.packed) launch_resident<0, 8, 2, 2, false, 1, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 8, 2, 2, false, 1>(g0, p0.resident_lds, stream);
    }
  } else {
    launch_route_topk(r.logits, a.M, r.num_experts, a.top_k, r.renormalize, r.topk_ids, r.topk_w, stream);
    if (shape == 2) {
      if (p0.packed) launch_resident<0, 8, 2, 2, false, 2, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 8, 2, 2, false, 2>(g0, p0.resident_lds, stream);
    } else {
      if (p0.packed) launch_resident<0, 4, 2, 8, false, 2, true>(g0, p0.resident_lds, stream);
      else launch_resident<0, 4, 2, 8, false, 2>(g0, p0.resident_lds, stream);
    }
  }
  g1.topk_w = r.topk_w;
  launch_stage<1>(g1, p1, stream);
  return true;
}

void launch_moe_gateup(const FusedMoeArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return;
  const GemmArgs g = gateup_args(a);
  launch_stage<0>(g, plan_stage<0>(g), stream);
}

// The linear part of a stage for one K slice (tensor-parallel ranks; the reference's
// moe_gateup_preact / moe_down_preact, src/c/vkernels/kernels/moe_fused.hpp:259-283):
// rows of `a` are a_stride wide and the slice starts at column k_base of each; w / w_scale
// are the rank's shard [E, rows, k_dim / 2] and [E, rows, k_dim / 32].  stage 0: rows =
// 2 * ncols, preact [EM, 2 * ncols] (gate columns, then up columns); stage 1: rows =
// ncols, preact [EM, ncols].  Routed rows are written, the others left as they are.
// Runs the decode kernel or the plain tile kernel (no workspace).  packed (optional): the
// shard in the prepacked form, which the decode kernels then read; w / w_scale may be null
// with it, and the call is then refused (false, nothing enqueued) where the decode kernels
// do not take it.
bool launch_moe_preact(int stage, const uint16_t* a, const uint8_t* w, const uint8_t* w_scale,
                       const int32_t* sorted_ids, const int32_t* expert_ids, float* preact, int M,
                       int a_stride, int ncols, int top_k, int EM, int k_base, int k_dim, int block_size,
                       hipStream_t stream, const uint8_t* packed, int num_experts) {
  if (M <= 0 || EM <= 0 || block_size <= 0) return true;
  GemmArgs g{};
  g.A = a + k_base;
  g.a_stride = a_stride;
  g.W = w;
  g.Ws = w_scale;
  if (packed != nullptr && num_experts > 0) {
    g.p_units = mx_units(stage, ncols);
    g.p_experts = num_experts;
    g.Wp = packed;
    g.Wpf = packed + mx_packed_body_bytes(num_experts, g.p_units, mx_kp(k_dim) / 128);
  }
  g.sorted_ids = sorted_ids;
  g.expert_ids = expert_ids;
  g.preact = preact;
  g.n_flat = M * top_k;
  g.top_k = top_k;
  g.K = k_dim;
  g.ncols = ncols;
  g.num_blocks = EM / block_size;
  g.block_size = block_size;
  const StagePlan pl = stage == 0 ? plan_stage<0>(g) : plan_stage<1>(g);
  if (w == nullptr && !(pl.packed && pl.variant == kMoeVariantResident)) return false;
  if (stage == 0) launch_stage<0>(g, pl, stream);
  else launch_stage<1>(g, pl, stream);
  return true;
}

// The second stage alone.  With a workspace (and packed weights) it runs as in the
// fused call: act split by a pass of its own, rows stored and summed per token.
void launch_moe_down(const FusedMoeArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return;
  GemmArgs g = down_args(a);
  const StagePlan pl = plan_stage<1>(g);
  const bool overwrite = (a.flags & 1u) != 0u;  // VK_HIP_MOE_OVERWRITE_OUT
  if (pl.variant != kMoeVariantResident) {
    if (a.w2_packed != nullptr && launch_moe_down_prepacked(a, stream)) return;
    Workspace w;
    if (carve_workspace(a, w) && g.K >= 512 && wide_kernel_ready<1>()) {
      const long long pieces = (long long)a.EM * split_row_k(a.ispp) / 8;
      hipLaunchKernelGGL(split_rows_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0,
                         stream, a.act, w.act_q, w.act_s, pieces, a.ispp);
      g.Aq = w.act_q;
      g.As = w.act_s;
      g.y = w.y;
      g.pos = w.pos;
      launch_fill_i32(w.pos, -1, a.M * a.top_k, stream);
      launch_stage<1>(g, pl, stream);
      launch_combine(w.y, w.pos, a.out, a.M, a.top_k, a.hidden, overwrite, stream);
      return;
    }
  }
  if (overwrite) launch_fill_i32(reinterpret_cast<int32_t*>(a.out), 0, a.M * a.hidden, stream);
  launch_stage<1>(g, pl, stream);
}

// Both stages.  With a workspace, a stage that runs as the tile kernel takes
// its rows already split: A by a pass of its own, act by the first stage's
// epilogue (which writes the bf16 act as well; the exact fallback reads it).
void launch_fused_moe(const FusedMoeArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.EM <= 0 || a.block_size <= 0) return;
  GemmArgs g0 = gateup_args(a);
  GemmArgs g1 = down_args(a);
  const StagePlan p0 = plan_stage<0>(g0), p1 = plan_stage<1>(g1);
  // prefill-sized batches on prepacked weights: the FP4-rate kernels of moe_prefill.hip
  if (a.w13_packed != nullptr && p0.variant != kMoeVariantResident &&
      p1.variant != kMoeVariantResident &&
      launch_fused_moe_prepacked(a, stream))
    return;
  // Without raw weights the decode kernels' packed forms take the call when both stages
  // are theirs, and the prepacked kernels any other (fused_moe_packed_only_ok has checked
  // that they can: the tile kernels below read raw weights).
  if (a.w13 == nullptr && (p0.variant != kMoeVariantResident || p1.variant != kMoeVariantResident)) {
    (void)launch_fused_moe_prepacked(a, stream);
    return;
  }
  Workspace w;
  bool combine = false;
  bool split_act_between = false;
  if (carve_workspace(a, w)) {
    // the wide kernel takes a stage that runs as a tile kernel with K >= 512
    const bool wide0 = p0.variant != kMoeVariantResident && g0.K >= 512 && wide_kernel_ready<0>();
    const bool wide1 = p1.variant != kMoeVariantResident && g1.K >= 512 && wide_kernel_ready<1>();
    if (wide0) {
      const long long pieces = (long long)a.M * split_row_k(a.hidden) / 8;
      hipLaunchKernelGGL(split_rows_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0,
                         stream, a.A, w.a_q, w.a_s, pieces, a.hidden);
      g0.Aq = w.a_q;
      g0.As = w.a_s;
    }
    if (wide1) {
      g1.Aq = w.act_q;
      g1.As = w.act_s;
      if (wide0) {  // the first stage's epilogue writes act in split form as well
        g0.actq = w.act_q;
        g0.actqs = w.act_s;
      } else {
        split_act_between = true;
      }
      // The second stage stores its rows and a last pass sums them per token (far
      // cheaper than one atomic per row and column).
      combine = true;
      g1.y = w.y;
      g1.pos = w.pos;
      launch_fill_i32(w.pos, -1, a.M * a.top_k, stream);
    }
  }
  const bool overwrite = (a.flags & 1u) != 0u;  // VK_HIP_MOE_OVERWRITE_OUT
  if (overwrite && !combine) {
    g0.zero_out = a.out;
    g0.zero_count = (long long)a.M * a.hidden;
  }
  launch_stage<0>(g0, p0, stream);
  if (split_act_between) {  // every sorted row, padding rows included (they hold old data)
    const long long pieces = (long long)a.EM * split_row_k(a.ispp) / 8;
    hipLaunchKernelGGL(split_rows_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream,
                       a.act, w.act_q, w.act_s, pieces, a.ispp);
  }
  launch_stage<1>(g1, p1, stream);
  if (combine) {
    launch_combine(w.y, w.pos, a.out, a.M, a.top_k, a.hidden, overwrite, stream);
  }
}

}  // namespace vk
