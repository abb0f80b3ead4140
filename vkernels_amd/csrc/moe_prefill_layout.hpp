// moe_prefill_layout.hpp — every byte offset the prefill kernel (moe_prefill.hip) forms, as
// pure functions of integers.  The kernel calls them; tests/test_prefill_layout.py compiles
// them for the host and walks all workgroups, wavefronts, lanes and K steps of a problem,
// checking that every offset stays inside the buffer it indexes and that the bytes a lane
// reads from LDS as its MFMA operand are the bytes of the row and K block it stands for.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifndef __HIPCC__
#ifndef __host__
#define __host__
#define __device__
#endif
#endif

namespace vk {

constexpr int kMxRows = 128;        // sorted rows per window
constexpr int kMxUnitRows = 128;    // weight rows per unit
constexpr int kMxWaves = 4;
constexpr int kMxRing = 3;          // K steps of split rows in LDS
constexpr int kMxStepBytes = 8704;  // prepacked bytes of one unit's K step: 8 KiB of codes + 512 of scales

// ring slot that holds the rows of K step `step`, register set that holds its weights
__host__ __device__ constexpr inline int mx_ring_slot(int step) { return step % kMxRing; }
__host__ __device__ constexpr inline int mx_weight_set(int step) { return step % 3; }

__host__ __device__ constexpr inline int mx_kp(int K) { return (K + 127) & ~127; }
__host__ __device__ constexpr inline int mx_units(int stage, int ncols) {
  return stage == 0 ? ncols / 64 : (ncols + kMxUnitRows - 1) / kMxUnitRows;
}
// Row of W (within an expert) that lane row n of tile t of `unit` multiplies; the
// caller checks it against the expert's row count (stage 1's last unit may be ragged).
__host__ __device__ constexpr inline int mx_weight_row(int stage, int ncols, int unit, int t, int n) {
  if (stage == 0) return (t >> 1) * ncols + unit * 64 + (t & 1) * 32 + n;
  return unit * kMxUnitRows + t * 32 + n;
}
__host__ __device__ constexpr inline int mx_window_rows(int block_size) {
  if (kMxRows % block_size == 0) return kMxRows;
  for (int rows = kMxRows; rows > 16; rows -= 16)
    if (block_size % rows == 0) return rows;
  return 16;
}

__host__ __device__ constexpr inline size_t mx_align256(size_t n) { return (n + 255) & ~(size_t)255; }

// ---- prepacked weights: [E][units][K steps] blocks of kMxStepBytes, then [E][units] flags ----
__host__ __device__ constexpr inline size_t mx_packed_body_bytes(int num_experts, int units, int nsteps) {
  return mx_align256((size_t)num_experts * (size_t)units * (size_t)nsteps * (size_t)kMxStepBytes);
}
__host__ __device__ constexpr inline size_t mx_packed_bytes(int num_experts, int units, int nsteps) {
  return mx_packed_body_bytes(num_experts, units, nsteps) + mx_align256((size_t)num_experts * (size_t)units);
}
// first byte of (expert, unit)'s K steps; a step past the end reads the last one again
__host__ __device__ constexpr inline size_t mx_unit_offset(int e, int units, int unit, int nsteps) {
  return ((size_t)e * (size_t)units + (size_t)unit) * (size_t)nsteps * (size_t)kMxStepBytes;
}
__host__ __device__ constexpr inline size_t mx_step_offset(int step, int nsteps) {
  return (size_t)(step < nsteps - 1 ? step : nsteps - 1) * (size_t)kMxStepBytes;
}
// byte of a step's block that load j (0 .. 7: the operand tiles, 16 bytes; 8: the scale
// bytes, 8 bytes) of `lane` starts at
__host__ __device__ constexpr inline int mx_weight_load_offset(int j, int lane) {
  return j < 8 ? (j >> 2) * 4096 + (j & 3) * 1024 + lane * 16 : 8192 + lane * 8;
}
__host__ __device__ constexpr inline size_t mx_flag_offset(int num_experts, int units, int nsteps, int e, int unit) {
  return mx_packed_body_bytes(num_experts, units, nsteps) + (size_t)e * (size_t)units + (size_t)unit;
}

// ---- split rows: row r = `terms` planes of kp bytes; 16-byte piece q of a plane's K step ----
// Copy operation (term, g) of a K step, issued by wavefront `wave`: lane (r, c) = (lane / 8,
// lane % 8) copies piece c ^ r of row (32 wave + 8 g + r) of the window to LDS position c
// of that row.  Source offset within the split rows (grow = the row's index there):
__host__ __device__ constexpr inline uint32_t mx_row_copy_lane_offset(size_t grow, int terms, int kp, int lane) {
  const int r = lane >> 3, c = lane & 7;
  return (uint32_t)(grow * (size_t)(terms * kp)) + 16u * (uint32_t)(c ^ r);
}
__host__ __device__ constexpr inline uint32_t mx_row_copy_step_offset(int term, int kp, int step, int nsteps) {
  return (uint32_t)(term * kp + (step < nsteps - 1 ? step : nsteps - 1) * 128);
}
// LDS destination of lane 0 of that copy (lane l lands 16 l bytes further)
__host__ __device__ constexpr inline int mx_slot_bytes(int terms) { return kMxRows * terms * 128; }
__host__ __device__ constexpr inline uint32_t mx_row_copy_lds(int step, int wave, int terms, int term, int g) {
  return (uint32_t)(mx_ring_slot(step) * mx_slot_bytes(terms) + ((wave * terms + term) * 32 + g * 8) * 128);
}
// ---- operand reads: lane (ln, hh) = (lane % 32, lane / 32) takes K block 2 half + hh of
// row ln of row tile m: 16-byte pieces 2 blk and 2 blk + 1, at positions (2 blk) ^ (ln & 7)
// and that ^ 1.  `which` = 2 half + (0: first piece, 1: second piece). ----
__host__ __device__ constexpr inline uint32_t mx_operand_lane_offset(int which, int ln, int hh) {
  const uint32_t pos0 = (uint32_t)(((2 * hh) ^ (ln & 7)) * 16);
  const uint32_t flip = which == 0 ? 0u : which == 1 ? 16u : which == 2 ? 64u : 80u;
  return (uint32_t)(ln * 128) + (pos0 ^ flip);
}
__host__ __device__ constexpr inline uint32_t mx_operand_tile_offset(int slot, int terms, int m, int term) {
  return (uint32_t)(slot * mx_slot_bytes(terms) + ((m * terms + term) * 32) * 128);
}
// ---- the K loop's schedule, as numbers: the kernel's counted waits and the host-side
// model of them (tests/prefill_layout_check.cpp) are built from these ----
// vector-memory operations a wavefront issues per K step: 4 row copies per term (8 rows
// x 128 bytes each, its row tile's 32 rows), 8 weight loads, 1 scale load
__host__ __device__ constexpr inline int mx_row_ops(int terms) { return 4 * terms; }
__host__ __device__ constexpr inline int mx_step_ops(int terms) { return mx_row_ops(terms) + 9; }
// groups of 4 MFMAs (one operand read each) per K step with `live` row tiles
__host__ __device__ constexpr inline int mx_step_groups(int live, int terms) { return 2 * live * terms; }
// The operations of step c + 2 are issued in groups 0 .. Q - 3 of step c, this many per
// group; the step's one wait (at most mx_step_ops outstanding: step c + 1 has landed, step
// c + 2 may be on its way) and barrier come at the end of group Q - 3.
__host__ __device__ constexpr inline int mx_ops_per_group(int live, int terms) {
  return (mx_step_ops(terms) + mx_step_groups(live, terms) - 3) / (mx_step_groups(live, terms) - 2);
}
__host__ __device__ constexpr inline int mx_wait_group(int live, int terms) { return mx_step_groups(live, terms) - 3; }

// ---- epilogue staging: a wavefront's own quarter of the ring ----
__host__ __device__ constexpr inline uint32_t mx_stage_base(int wave, int terms) {
  return (uint32_t)(wave * (kMxRing * mx_slot_bytes(terms) / kMxWaves));
}
constexpr int kMxActPitch = 144;  // stage 0: 64 bf16 of a row + 16 bytes (rows stay 16-byte aligned)
constexpr int kMxYPitch = 272;    // stage 1: 64 floats of a row + 16 bytes

}  // namespace vk
