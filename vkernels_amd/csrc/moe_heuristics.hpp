// moe_heuristics.hpp — tile shapes of the MoE grouped GEMMs for gfx950.
//
// Same role as the GEMM candidate table of the reference
// (src/c/vkernels/kernels/common/heuristics.hpp:20-61), which has no MoE
// entries of its own: a small table of launch shapes and a pure function
// that picks one from the problem size on the host.
#pragma once

namespace vk {

struct MoeTile {
  int waves;  // wavefronts per workgroup
  int nt;     // 16-row weight tiles per wavefront
  int mt;     // 16-row activation tiles per pass
};

}  // namespace vk
