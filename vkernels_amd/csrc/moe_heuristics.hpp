// moe_heuristics.hpp — launch shapes of the MoE grouped GEMMs for gfx950.
//
// Same role as the GEMM candidate table of the reference
// (src/c/vkernels/kernels/common/heuristics.hpp:20-61), which has no MoE
// entries of its own: a small table of launch shapes and a pure function
// that picks one from the problem size on the host.
#pragma once

namespace vk {

enum { kMoeVariantLds = 0, kMoeVariantResident = 2 };

struct MoeTile {
  int variant;  // kMoeVariantResident: one workgroup per compute unit, the
                // activation rows of a run resident in LDS (decode);
                // kMoeVariantLds: activation rows staged through LDS chunk by chunk
  int waves;    // wavefronts per workgroup
  int nt;       // 16-row weight tiles per wavefront
  int depth;    // K steps in flight per wavefront (resident variant)
};

// n_flat = tokens * top_k routed rows in the call, K / ncols the GEMM's
// reduction and output widths, stage 0 = gate/up, 1 = down.  The number of
// experts is not known to the launcher, so the split is on the routed rows
// alone: a decode batch leaves most experts with at most one 16-row tile.
//
// Decode: the units of a run are shared by (compute units / runs) workgroups
// of 8 wavefronts, so a stage wants at least ~3 units per wavefront or the
// last round leaves most wavefronts idle.  Gate/up units are a gate tile and
// its up tile (nt = 2, ispp / 16 units per expert); the down stage, with half
// the weight rows, takes single tiles (nt = 1) and keeps the bytes in flight
// per wavefront with a deeper pipeline.
inline MoeTile pick_moe_tile(int n_flat, int K, int ncols, int stage) {
  (void)K;
  (void)ncols;
  if (n_flat <= 512) {
    if (stage == 1) return MoeTile{kMoeVariantResident, 8, 1, 8};
    return MoeTile{kMoeVariantResident, 8, 2, 4};
  }
  return MoeTile{kMoeVariantLds, 4, 4, 0};
}

}  // namespace vk
