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
// and, for every number of live row tiles, the K loop's schedule of one wavefront (the
// kernel's loop structure restated with the schedule functions of the same header): every
// vector-memory operation in program order against the counted waits, the LDS reads
// against the waits for them, the barriers, and the ring slots and weight register sets
// they touch:
//   - when an MFMA uses a step's weights, a wait has forced that step's loads to land;
//   - when an operand is read from a ring slot, every wavefront's copies of that step have
//     landed (each wavefront waited for its own, then a barrier);
//   - when a copy is issued into a ring slot, every read of the step it overwrites has
//     completed in every wavefront (a wait for the LDS reads, then a barrier);
//   - when a load is issued into a weight register set, the MFMAs of the step it
//     overwrites are behind it;
//   - before the epilogue writes its staging area over the ring, nothing is in flight.
// Usage: prefill_layout_check stage terms K ncols num_experts rows ; exit status 0 = all hold.
// Built with -DVK_LAYOUT_BREAK_WAIT the model's wait lets one operation too many stay
// outstanding, which the walk must notice (the test of the test).
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

// ---- the schedule of one wavefront ----------------------------------------------------------
namespace {

struct Event {
  enum Kind { kCopy, kLoad, kWait, kLdsWait, kBarrier, kRead, kUse, kStaging } kind;
  int step;  // K step the operation belongs to (copies, loads, reads, uses)
  int n;     // kWait: operations that may stay outstanding
};

// Program order of the K loop and what follows it, as tile_mx_kernel issues it.
std::vector<Event> schedule(int terms, int live, int nsteps) {
  const int ops = mx_step_ops(terms), rows = mx_row_ops(terms);
  const int Q = mx_step_groups(live, terms), per = mx_ops_per_group(live, terms);
  std::vector<Event> ev;
  auto issue = [&](int step, int k) { ev.push_back({k < rows ? Event::kCopy : Event::kLoad, step, 0}); };
  // prologue: the operations of steps 0 and 1, a wait that leaves step 1's outstanding, a barrier,
  // the reads of the first two groups
  for (int k = 0; k < ops; ++k) issue(0, k);
  for (int k = 0; k < ops; ++k) issue(1, k);
#ifdef VK_LAYOUT_BREAK_WAIT
  ev.push_back({Event::kWait, 0, ops + 1});
#else
  ev.push_back({Event::kWait, 0, ops});
#endif
  ev.push_back({Event::kBarrier, 0, 0});
  ev.push_back({Event::kRead, 0, 0});
  ev.push_back({Event::kRead, 0, 0});
  for (int c = 0; c < nsteps; ++c) {
    int issued = 0;
    for (int q = 0; q < Q; ++q) {
      ev.push_back({Event::kUse, c, 0});                                     // the group's MFMAs
      ev.push_back({Event::kRead, q + 2 < Q ? c : c + 1, 0});                // the operand of group q + 2
      if (q < Q - 2) {
        for (int k = 0; k < per; ++k)
          if (issued + k < ops) issue(c + 2, issued + k);
        issued += per;
      }
      if (q == mx_wait_group(live, terms)) {
        ev.push_back({Event::kWait, c, ops});
        ev.push_back({Event::kLdsWait, c, 0});
        ev.push_back({Event::kBarrier, c, 0});
      }
    }
  }
  ev.push_back({Event::kWait, nsteps, 0});   // the loads issued past the last step land
  ev.push_back({Event::kBarrier, nsteps, 0});
  ev.push_back({Event::kStaging, nsteps, 0});
  return ev;
}

// Walks the schedule; 0 = every rule of the header comment holds.
int check_schedule(int terms, int live, int nsteps) {
  const std::vector<Event> ev = schedule(terms, live, nsteps);
  const int ops = mx_step_ops(terms);
  std::vector<int> vm;          // issue positions (indices into ev) of the vector-memory operations, in order
  size_t landed = 0;            // operations known to have landed (a wait forced them)
  // per K step: operations issued, operations landed, landed-and-behind-a-barrier (every wavefront's),
  // reads issued, reads completed, completed-and-behind-a-barrier, MFMA groups issued
  const int S = nsteps + 4;
  std::vector<int> issued(S, 0), done(S, 0), done_all(S, 0), reads(S, 0), reads_done(S, 0), reads_done_all(S, 0), uses(S, 0);
  std::vector<int> step_of;     // step of each vector-memory operation
  for (size_t i = 0; i < ev.size(); ++i) {
    const Event& e = ev[i];
    switch (e.kind) {
      case Event::kCopy: {
        // the slot held step e.step - kMxRing: all its reads complete everywhere
        const int old = e.step - kMxRing;
        if (old >= 0) {
          CHECK(reads_done_all[old] == reads[old], "terms %d live %d nsteps %d: a copy of step %d is issued while "
                "reads of step %d may be under way", terms, live, nsteps, e.step, old);
          CHECK(uses[old] > 0 || old >= nsteps, "copy before the step it overwrites was used");
        }
        CHECK(mx_ring_slot(e.step) == mx_ring_slot(e.step + kMxRing), "ring");
        vm.push_back((int)i);
        step_of.push_back(e.step);
        ++issued[e.step];
        break;
      }
      case Event::kLoad: {
        const int old = e.step - 3;  // the register set's previous step: its MFMAs are all issued
        if (old >= 0 && old < nsteps)
          CHECK(uses[old] == mx_step_groups(live, terms), "terms %d live %d nsteps %d: a weight load of step %d is "
                "issued before the MFMAs of step %d", terms, live, nsteps, e.step, old);
        CHECK(mx_weight_set(e.step) == mx_weight_set(e.step + 3), "sets");
        vm.push_back((int)i);
        step_of.push_back(e.step);
        ++issued[e.step];
        break;
      }
      case Event::kWait: {
        const size_t must = vm.size() > (size_t)e.n ? vm.size() - (size_t)e.n : 0;
        for (; landed < must; ++landed) ++done[step_of[landed]];
        break;
      }
      case Event::kLdsWait:
        for (int s = 0; s < S; ++s) reads_done[s] = reads[s];
        break;
      case Event::kBarrier:
        for (int s = 0; s < S; ++s) {
          if (done[s] == issued[s]) done_all[s] = done[s];
          reads_done_all[s] = reads_done[s];
        }
        break;
      case Event::kRead:
        // (a read of the step after the last only fetches an operand nobody multiplies, but
        // it still reads the ring: the same rule)
        CHECK(issued[e.step] == ops && done_all[e.step] == ops, "terms %d live %d nsteps %d: an operand of step %d "
              "is read before every wavefront's copies of it have landed", terms, live, nsteps, e.step);
        ++reads[e.step];
        break;
      case Event::kUse:
        CHECK(issued[e.step] == ops && done[e.step] == ops, "terms %d live %d nsteps %d: step %d's weights are used "
              "before a wait has let them land", terms, live, nsteps, e.step);
        ++uses[e.step];
        break;
      case Event::kStaging:
        CHECK(landed == vm.size(), "terms %d live %d nsteps %d: operations in flight when the epilogue starts",
              terms, live, nsteps);
        for (int s = 0; s < S; ++s)
          CHECK(reads_done_all[s] == reads[s] || reads[s] == 0 || s >= nsteps,
                "reads of step %d outstanding at the epilogue", s);
        break;
    }
  }
  // every K step was multiplied, with all its groups, and every step's operations were issued once
  for (int c = 0; c < nsteps; ++c) CHECK(uses[c] == mx_step_groups(live, terms) && issued[c] == ops, "step %d", c);
  CHECK(mx_ops_per_group(live, terms) * (mx_step_groups(live, terms) - 2) >= ops, "a step's operations do not fit its groups");
  return 0;
}

}  // namespace

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
  // ---- the K loop's schedule: every number of live row tiles the kernel compiles, the
  // problem's own K steps and the shortest loops ----
  for (int live = 1; live <= 4; ++live) {
    if (live == 1 && terms == 1) continue;  // (one plane per row: the kernel runs two live tiles then)
    for (int steps : {1, 2, 3, 4, 5, 7, nsteps})
      if (check_schedule(terms, live, steps) != 0) return 1;
  }
  return 0;
}
