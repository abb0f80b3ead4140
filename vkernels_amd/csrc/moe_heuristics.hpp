// moe_heuristics.hpp — launch shapes of the MoE grouped GEMMs for gfx950, as data.
//
// Same layering as the reference's GEMM candidates
// (src/c/vkernels/kernels/common/heuristics.hpp:20-61, which has no MoE entries of its
// own): the table of shapes that are compiled and were swept, and a selector that only
// ever returns entries of it.  The selector is consulted after the tuning store
// (moe_tuning.hpp), the way the reference's selectors are (core/tuning.hpp:1-9).
#pragma once

#include <cstddef>

namespace vk {

enum { kMoeVariantLds = 0, kMoeVariantResident = 2, kMoeVariantResidentKSplit = 3, kMoeVariantChunked = 4 };

struct MoeTile {
  int variant;  // kMoeVariantResident: one workgroup per compute unit, the
                // activation rows of a run resident in LDS (decode);
                // kMoeVariantResidentKSplit: the same, the K steps of a unit shared between
                // the wavefronts that would otherwise have none (a handful of rows);
                // kMoeVariantChunked: the decode kernel of the prepacked form that holds the
                // rows a chunk of K at a time (rows of any K; blocks of 16 or of 32 rows,
                // the 32 rows of a block in one pass over the expert's weights);
                // kMoeVariantLds: the tile kernels (rows staged through LDS)
  int waves;    // wavefronts per workgroup
  int nt;       // 16-row weight tiles per wavefront
  int depth;    // K steps in flight per wavefront (resident variant)
};

inline bool operator==(const MoeTile& a, const MoeTile& b) {
  return a.variant == b.variant && a.waves == b.waves && a.nt == b.nt && a.depth == b.depth;
}

// Every shape a stage can be launched at: the instantiations of the resident kernel
// (X(stage, wavefronts, tiles, depth) — moe_gemm.hip instantiates exactly these) and
// the tile kernels as one more entry.  The sweep (vkernels_amd/tune_moe.py) times each
// of these for a stage and a problem size.
#define VK_RESIDENT_VARIANTS(X) \
  X(0, 8, 2, 2) X(0, 8, 2, 4) X(0, 8, 2, 6) X(0, 4, 2, 4) X(0, 4, 2, 8) \
  X(1, 8, 2, 4) X(1, 8, 1, 4) X(1, 8, 1, 6) X(1, 8, 1, 8) X(1, 8, 1, 12)
// ... and of its K-split form (every one is also in the list above: a plan that cannot
// split K falls back to the same shape there).
#define VK_KSPLIT_VARIANTS(X) X(0, 8, 2, 4) X(0, 8, 2, 6) X(1, 8, 1, 8) X(1, 8, 2, 4)
// ... and of the chunked kernel (prepacked form only; 8 wavefronts).
#define VK_CHUNKED_VARIANTS(X) X(0, 8, 2, 2) X(0, 8, 2, 4) X(1, 8, 1, 2) X(1, 8, 1, 4)

struct MoeTileCandidate {
  int stage;
  MoeTile tile;
};

inline const MoeTileCandidate* moe_tile_candidates(size_t* count) {
  static const MoeTileCandidate table[] = {
#define VK_CANDIDATE(S_, W_, NT_, D_) {S_, {kMoeVariantResident, W_, NT_, D_}},
      VK_RESIDENT_VARIANTS(VK_CANDIDATE)
#undef VK_CANDIDATE
#define VK_CANDIDATE(S_, W_, NT_, D_) {S_, {kMoeVariantResidentKSplit, W_, NT_, D_}},
      VK_KSPLIT_VARIANTS(VK_CANDIDATE)
#undef VK_CANDIDATE
#define VK_CANDIDATE(S_, W_, NT_, D_) {S_, {kMoeVariantChunked, W_, NT_, D_}},
      VK_CHUNKED_VARIANTS(VK_CANDIDATE)
#undef VK_CANDIDATE
      {0, {kMoeVariantLds, 4, 4, 0}},
      {1, {kMoeVariantLds, 4, 4, 0}},
  };
  *count = sizeof(table) / sizeof(table[0]);
  return table;
}

inline bool is_moe_tile_candidate(int stage, const MoeTile& tile) {
  size_t n = 0;
  const MoeTileCandidate* table = moe_tile_candidates(&n);
  for (size_t i = 0; i < n; ++i)
    if (table[i].stage == stage && table[i].tile == tile) return true;
  return false;
}

// Routed rows up to which a call runs the resident (decode) kernels: beyond, most
// experts have several 16-row passes and the tile kernels, which keep a 128-row window
// per workgroup, read each weight byte once per window instead of once per pass.
constexpr int kMoeDecodeMaxRows = 512;
// A caller that gives the prepacked weights also says how many experts they hold, and
// what decides between the families is rows per expert, not rows: a pass per 16 rows of an
// expert against a window per expert.  With blocks of 16 the decode kernels then take
// calls of up to this many routed rows per expert as well (measured on the prepacked
// form, decode against tile kernels: 600 rows on 64 experts, 9.4 each, 164 against 195 us;
// 636 rows, 9.9 each, 183 against 194 us; 1024 rows on 128 experts with a few popular ones,
// 8 each, 226 against 255 us -- but 1280 rows there, 10 each, 272 against 256 us; 1530 on
// 64, 24 each, 263 against 204 us; 1024 on 32: 199 against 156 us) -- as long as the runs
// (a block of 16 per pass, one more per expert for its partly filled one) fit the run list.
constexpr int kMoeDecodeRowsPerExpert = 9;
constexpr int kMoeMaxRuns = 512;  // runs the decode kernel lists in LDS

inline int moe_decode_max_rows(int packed_experts) {
  if (packed_experts <= 0) return kMoeDecodeMaxRows;
  const long long by_expert = (long long)kMoeDecodeRowsPerExpert * packed_experts;
  const long long by_runs = 16ll * (kMoeMaxRuns - packed_experts);
  const long long m = by_expert < by_runs ? by_expert : by_runs;
  return m > kMoeDecodeMaxRows ? (int)m : kMoeDecodeMaxRows;
}

// Blocks of 32 rows on the prepacked form (the chunked decode kernel multiplies both 16-row
// tiles of a block with every weight register): up to this many routed rows per expert
// (measured against the prepacked tile kernels in blocks of 128, us a step: 32 experts,
// 1024 rows, 32 each, 144 against 160, and 1200 rows, 37.5 each, 175 against 168; 64
// experts, 1800 rows, 28 each, 193 against 207, 2100 rows, 33 each, 214 against 216, 2520
// rows, 39 each, 248 against 227; 128 experts with a few popular ones, 2048 rows, 269
// against 277; 256 experts of 7168 x 2048, 4000 rows, 16 each, 1157 against 1304, but 8000
// rows, 31 each, where four experts in ten have a second block, 1687 against 1397).
constexpr int kMoeDecodeRowsPerExpert32 = 28;
// Routed rows up to which the first stage's decode kernel routes or aligns for itself
// (blocks of 16 only).
constexpr int kMoeRoutedMaxRows = 256;

inline int moe_decode_max_rows32(int packed_experts) {
  if (packed_experts <= 0) return kMoeDecodeMaxRows;
  const long long by_expert = (long long)kMoeDecodeRowsPerExpert32 * packed_experts;
  const long long by_runs = 32ll * (kMoeMaxRuns - packed_experts);
  const long long m = by_expert < by_runs ? by_expert : by_runs;
  return m > kMoeDecodeMaxRows ? (int)m : kMoeDecodeMaxRows;
}

// One row of the decision table: the first row whose bounds hold decides.
struct MoeTileRule {
  int stage;
  int max_rows;  // n_flat <= max_rows
  int max_k;     // K <= max_k
  MoeTile tile;
};

// n_flat = tokens * top_k routed rows in the call, K / ncols the GEMM's reduction and
// output widths, stage 0 = gate/up, 1 = down.  Neither the number of experts nor the
// number of runs is known to the launcher (EM may be the caller's upper bound), so the
// split between the kernel families is on the routed rows alone.
//
// Decode: the units of a run are shared by (compute units / runs) workgroups of 8
// wavefronts, so a stage wants at least ~3 units per wavefront or the last of them leaves
// most wavefronts idle.  Gate/up units are a gate tile and its up tile (nt = 2,
// ispp / 16 units per expert); the down stage, with half the weight rows, takes single
// tiles (nt = 1) and keeps the bytes in flight per wavefront with a deeper pipeline.
// Rows (each from the sweep table profiles/moe_decode_tile_sweep.md):
//  - the shallowest pipelines of the table (with K <= 1024 a unit is a few steps long, and
//    steps in flight past its end are wasted loads: 256x512x8x2 at T = 64, 8.7 against 9.2 us;
//    with longer rows the depth hardly matters);
//  - 3072 < K <= 4096 (4096x1536x64x6 gate/up): the rows of a pass fit LDS and registers
//    only with 4 wavefronts per workgroup (34 against 69 us at T = 1, 97 against 185 us
//    at T = 32 for the tile kernel, which is what runs beyond K = 4096);
//  - down stage: single tiles, four K steps in flight, at every size (units of two tiles
//    were 4 to 5 % faster up to 24 rows while a lane's epilogue held four columns of one row;
//    with the rows as the matrix cores' first operand a lane holds one column of four rows,
//    and two tiles are 5 to 20 % behind there: 2880x2880x32x4 at T = 3, 20.2 against 16.7 us
//    on the prepacked form; six steps in flight are 1 to 3 % behind four at most points);
//  - otherwise (8, 2, 2) / (8, 1, 4), within 5 % of the best of every other point swept:
//    with 128 experts and 32 tokens or more, uniformly routed, the 4-wavefront shapes
//    are 3 to 5 % faster for gate/up; the number of runs that makes it so is not known
//    here, and with skewed routing (27 active experts of 128) the same shape is much
//    slower, so that choice is left to the tuning store.
//
// A single token or two: when the units of all rows (at most n_flat runs) are fewer than
// half the wavefronts of the device, a wavefront has one unit or none, and a unit is a chain
// of K / 128 dependent steps, a few in flight.  The K-split form gives the idle wavefronts a
// part of K each.  Only the shapes whose rows of K values need 8 wavefronts to stage have it
// (with 4 wavefronts, K up to 4096, all of K takes longer to stage than the shorter chains
// save: 4096x1536x64x6 at T = 1, 32.0 against 28.4 us).
constexpr int kMoeComputeUnits = 256;  // of the device the rules were swept on

// packed: the stage reads the prepacked form (its decode kernels have no scale block in
// LDS and fewer registers in use, so their best shapes are swept separately).
// packed_experts: their number when the call also comes in blocks of 16 or 32 (else 0): the
// decode range then follows moe_decode_max_rows.
// block_rows: the alignment's block size.  Blocks of 32 on the prepacked form go to the
// chunked kernel, a block a pass; so do rows of a K the resident kernel cannot hold.
inline MoeTile pick_moe_tile(int n_flat, int K, int ncols, int stage, bool packed = false,
                             int packed_experts = 0, int block_rows = 16) {
  // (four K steps in flight in both stages: for gate/up level with two up to 8 rows per
  // expert and 1 to 4 % ahead beyond -- 4096x1536x64x6 in blocks of 32 at T = 255: 98.8
  // against 101.9 us, 2880x2880x32x4: 75.3 against 78.3 us)
  const MoeTile chunked = MoeTile{kMoeVariantChunked, 8, stage == 0 ? 2 : 1, 4};
  if (packed && block_rows == 32)
    return n_flat <= moe_decode_max_rows32(packed_experts) ? chunked : MoeTile{kMoeVariantLds, 4, 4, 0};
  const int max_rows = moe_decode_max_rows(packed ? packed_experts : 0);
  // (on the prepacked form the 8-wavefront K-split shape also holds rows of K up to 4096)
  if (packed && stage == 0 && n_flat <= kMoeDecodeMaxRows && K > 3072 && K <= 4096 &&
      (long long)n_flat * (ncols / 16) <= (long long)kMoeComputeUnits * 4)
    return MoeTile{kMoeVariantResidentKSplit, 8, 2, 4};
  if (n_flat <= kMoeDecodeMaxRows && K >= 1024 && K <= 3072) {
    const long long spare = (long long)kMoeComputeUnits * 4;  // half of 8 wavefronts per compute unit
    if (stage == 0 && (long long)n_flat * (ncols / 16) <= spare)
      return MoeTile{kMoeVariantResidentKSplit, 8, 2, 4};
    if (stage == 1 && (long long)n_flat * (ncols / 16) <= spare)
      return MoeTile{kMoeVariantResidentKSplit, 8, 1, 8};
    if (stage == 1 && (long long)n_flat * (ncols / 32) <= spare)
      return MoeTile{kMoeVariantResidentKSplit, 8, 2, 4};
  }
  const MoeTileRule rules[] = {
      {0, max_rows, packed ? 4096 : 3072, {kMoeVariantResident, 8, 2, 2}},  // (the prepacked form's rows of a pass: K <= 4096)
      {0, max_rows, 4096, {kMoeVariantResident, 4, 2, 8}},
      {1, max_rows, 3072, {kMoeVariantResident, 8, 1, 4}},
  };
  for (const MoeTileRule& r : rules)
    if (r.stage == stage && n_flat <= r.max_rows && K <= r.max_k) return r.tile;
  if (packed && n_flat <= max_rows) return chunked;  // rows of any K
  return MoeTile{kMoeVariantLds, 4, 4, 0};
}

// Alignment block the library's kernels like best for a batch of M tokens routed to
// top_k experts each.  Decode kernel: a pass per 16 rows, and blocks of 16 tell it the
// passes of every expert exactly and pad least.  Tile kernels: a workgroup takes a
// window of 128 sorted rows of one expert, so blocks of 128 give every expert windows of
// its own (0.5 to 8 % faster than blocks of 64 from 16 to 770 rows per expert).
// packed_experts, hidden, ispp: the number of (local) experts and the layer's widths when
// the caller gives the prepacked weights, 0 otherwise.  On that form, beyond the rows of
// the routed forms (which want blocks of 16), blocks of 32 and the chunked decode kernel
// up to kMoeDecodeRowsPerExpert32 rows per expert: an expert with 17 to 32 rows costs one
// pass over its weights, not two (us a step, blocks of 16 / 32 / 128: 32 experts, 512
// rows, 124 / 111 / 142; 64 experts, 510 rows, 139 / 138 / 144, and 1530 rows, - / 181 /
// 201; 128 experts with a few popular ones, 1152 rows, 244 / 205 / 246).
inline int moe_default_block_size(int M, int top_k, int packed_experts = 0, int hidden = 0, int ispp = 0) {
  const long long n = (long long)M * (long long)top_k;
  if (n <= kMoeRoutedMaxRows) return 16;
  if (packed_experts > 0 && hidden > 0 && ispp > 0 && n <= moe_decode_max_rows32(packed_experts) &&
      hidden % 64 == 0 && ispp % 64 == 0)
    return 32;
  return n <= kMoeDecodeMaxRows ? 16 : 128;
}

}  // namespace vk
