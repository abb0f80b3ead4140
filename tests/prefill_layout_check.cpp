// Host-side walk over every address the prefill kernel forms (the functions of
// vkernels_amd/csrc/moe_prefill_layout.hpp, compiled for the CPU): for a problem
// (stage, terms, K, ncols, experts, rows) it visits all (expert, unit, K step, load, lane)
// and (row, term, K step, copy, lane) and (slot, row tile, term, half, lane) and checks
//   - every weight load lies inside the prepacked buffer, every flag inside its tail;
//   - every row copy reads inside the split rows and lands inside its slot of the ring,
//     no two lanes of a K step landing on the same bytes;
//   - the 32 bytes a lane reads as its operand are K block (2 half + hh) of row ln of its
//     row tile and term: the copy's XOR rotation and the read's undo each other;
//   - the epilogue's staging area lies inside the wavefront's quarter of the ring.
// Usage: prefill_layout_check stage terms K ncols num_experts rows ; exit status 0 = all hold.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "moe_prefill_layout.hpp"

using namespace vk;

#define CHECK(cond, ...)                                  \
  do {                                                    \
    if (!(cond)) {                                        \
      std::fprintf(stderr, "FAILED %s: ", #cond);         \
      std::fprintf(stderr, __VA_ARGS__);                  \
      std::fprintf(stderr, "\n");                         \
      return 1;                                           \
    }                                                     \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 7) return 2;
  const int stage = std::atoi(argv[1]), terms = std::atoi(argv[2]), K = std::atoi(argv[3]);
  const int ncols = std::atoi(argv[4]), E = std::atoi(argv[5]), rows = std::atoi(argv[6]);
  const int kp = mx_kp(K), nsteps = kp / 128, units = mx_units(stage, ncols);
  const size_t packed = mx_packed_bytes(E, units, nsteps);
  const size_t body = mx_packed_body_bytes(E, units, nsteps);
  const size_t split_bytes = (size_t)rows * (size_t)terms * (size_t)kp;
  const int ring = kMxRing * mx_slot_bytes(terms);
  CHECK(ring <= 160 * 1024 - 2048, "ring %d", ring);
  CHECK(kp >= K && kp % 128 == 0 && kp - K < 128, "kp %d", kp);

  // ---- weights ----
  for (int e : {0, E / 2, E - 1})
    for (int unit = 0; unit < units; ++unit) {
      const size_t u0 = mx_unit_offset(e, units, unit, nsteps);
      for (int step = 0; step < nsteps + 2; ++step)  // the pipeline asks for two steps past the end
        for (int j = 0; j < 9; ++j)
          for (int lane = 0; lane < 64; ++lane) {
            const size_t off = u0 + mx_step_offset(step, nsteps) + (size_t)mx_weight_load_offset(j, lane);
            CHECK(off + (j < 8 ? 16 : 8) <= body, "weight load e=%d unit=%d step=%d j=%d lane=%d", e, unit, step, j, lane);
          }
      const size_t f = mx_flag_offset(E, units, nsteps, e, unit);
      CHECK(f >= body && f < packed, "flag e=%d unit=%d", e, unit);
      // every weight row of the unit's tiles is a row of the expert or past its end (ragged last unit)
      for (int t = 0; t < 4; ++t)
        for (int n = 0; n < 32; ++n) {
          const int r = mx_weight_row(stage, ncols, unit, t, n);
          const int rows_w = stage == 0 ? 2 * ncols : ncols;
          CHECK(r >= 0 && (r < rows_w || (stage == 1 && unit == units - 1)), "weight row %d of %d", r, rows_w);
        }
    }
  // the bytes of one step's block are each loaded exactly once
  {
    std::vector<int> hit(kMxStepBytes, 0);
    for (int j = 0; j < 9; ++j)
      for (int lane = 0; lane < 64; ++lane)
        for (int b = 0; b < (j < 8 ? 16 : 8); ++b) ++hit[mx_weight_load_offset(j, lane) + b];
    for (int b = 0; b < kMxStepBytes; ++b) CHECK(hit[b] == 1, "byte %d of a step loaded %d times", b, hit[b]);
  }

  // ---- row copies and operand reads ----
  // LDS model: for every byte of a slot, which (row of the window, term, byte of the K step) it holds
  const int slot_bytes = mx_slot_bytes(terms);
  for (size_t grow : {(size_t)0, (size_t)rows / 2, (size_t)rows - 1})
    for (int step = 0; step < nsteps + 2; ++step)
      for (int term = 0; term < terms; ++term)
        for (int lane = 0; lane < 64; ++lane) {
          const size_t src = (size_t)mx_row_copy_lane_offset(grow, terms, kp, lane) +
                             mx_row_copy_step_offset(term, kp, step, nsteps);
          CHECK(src + 16 <= split_bytes, "row copy source grow=%zu step=%d term=%d lane=%d", grow, step, term, lane);
        }
  CHECK((unsigned long long)rows * terms * kp < (1ull << 32), "split rows beyond 32-bit offsets");
  for (int step = 0; step < 4; ++step) {
    std::vector<int> row_of(slot_bytes, -1), term_of(slot_bytes, -1), byte_of(slot_bytes, -1);
    const int base = (step % kMxRing) * slot_bytes;
    for (int wave = 0; wave < kMxWaves; ++wave)
      for (int term = 0; term < terms; ++term)
        for (int g = 0; g < 4; ++g)
          for (int lane = 0; lane < 64; ++lane) {
            const int dst = (int)mx_row_copy_lds(step, wave, terms, term, g) + 16 * lane - base;
            CHECK(dst >= 0 && dst + 16 <= slot_bytes, "copy lands outside its slot: %d", dst);
            const int r = lane >> 3, c = lane & 7;
            // piece of the K step this lane fetched (the source offset within the row's plane)
            const int piece = (int)(mx_row_copy_lane_offset(0, terms, kp, lane) / 16);
            CHECK(piece == (c ^ r), "piece");
            for (int b = 0; b < 16; ++b) {
              CHECK(row_of[dst + b] == -1, "two copies land on byte %d of the slot", dst + b);
              row_of[dst + b] = wave * 32 + g * 8 + r;
              term_of[dst + b] = term;
              byte_of[dst + b] = piece * 16 + b;
            }
          }
    for (int b = 0; b < slot_bytes; ++b) CHECK(row_of[b] >= 0, "byte %d of the slot is never written", b);
    for (int m = 0; m < 4; ++m)
      for (int term = 0; term < terms; ++term)
        for (int half = 0; half < 2; ++half)
          for (int lane = 0; lane < 64; ++lane) {
            const int ln = lane & 31, hh = lane >> 5;
            for (int part = 0; part < 2; ++part) {
              const int off = (int)mx_operand_lane_offset(2 * half + part, ln, hh) +
                              (int)mx_operand_tile_offset(step % kMxRing, terms, m, term) - base;
              CHECK(off >= 0 && off + 16 <= slot_bytes, "operand read outside the slot");
              for (int b = 0; b < 16; ++b) {
                CHECK(row_of[off + b] == m * 32 + ln && term_of[off + b] == term, "operand read: wrong row or term");
                // K block (2 half + hh) of 32 values = 32 bytes of the plane's K step
                CHECK(byte_of[off + b] == (2 * half + hh) * 32 + part * 16 + b, "operand read: wrong K bytes");
              }
            }
          }
  }
  // ---- epilogue staging ----
  for (int wave = 0; wave < kMxWaves; ++wave) {
    const int lo = (int)mx_stage_base(wave, terms);
    const int hi = wave + 1 < kMxWaves ? (int)mx_stage_base(wave + 1, terms) : ring;
    const int need = stage == 0 ? 31 * kMxActPitch + 128 : 31 * kMxYPitch + 256;
    CHECK(lo % 16 == 0 && lo + need <= hi, "staging area of wavefront %d: %d bytes in [%d, %d)", wave, need, lo, hi);
  }
  CHECK(kMxActPitch % 16 == 0 && kMxYPitch % 16 == 0, "pitch");
  return 0;
}
