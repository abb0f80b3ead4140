// launch_overhead.hip — what one launch of the decode kernel's shape costs on this device
// apart from its work: an (almost) empty kernel, one workgroup of 512 threads per compute
// unit and 120 KB of dynamic LDS, timed between HIP events, (a) as it is, (b) with a few
// bytes of scratch memory per lane, (c) launched cooperatively, (d) launched cooperatively
// with one grid-wide sync (thread 0's 100 MHz clock: last workgroup in -> last one out).
//
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops vkernels_amd/microbench/launch_overhead.hip -o /tmp/launch_overhead
//   /tmp/launch_overhead
#include <hip/hip_cooperative_groups.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <vector>

namespace cg = cooperative_groups;

#define CHECK(call)                                                                        \
  do {                                                                                     \
    const hipError_t err_ = (call);                                                        \
    if (err_ != hipSuccess) {                                                              \
      std::fprintf(stderr, "%s line %d: %s\n", #call, __LINE__, hipGetErrorString(err_)); \
      return 1;                                                                            \
    }                                                                                      \
  } while (0)

constexpr int kMaxWorkgroups = 1024;
__device__ unsigned long long g_stamp[kMaxWorkgroups][2];  // entry, after the sync

template <bool SCRATCH, bool SYNC>
__global__ __launch_bounds__(512) void empty_kernel(unsigned* sink, int index) {
  extern __shared__ unsigned lds[];
  if (threadIdx.x == 0) g_stamp[blockIdx.x][0] = wall_clock64();
  unsigned acc = threadIdx.x;
  if (SCRATCH) {
    volatile unsigned priv[8];
    for (int i = 0; i < 8; ++i) priv[i] = acc + i;
    acc = priv[index & 7];
  }
  lds[threadIdx.x] = acc;
  if (SYNC) {
    sink[blockIdx.x * 64 + (threadIdx.x & 63)] = acc;  // something for the sync to make visible
    cg::this_grid().sync();
    if (threadIdx.x == 0) g_stamp[blockIdx.x][1] = wall_clock64();
    if (sink[((blockIdx.x + 1) % gridDim.x) * 64] == 0x12345678u) sink[0] = lds[0];
  }
  if (acc == 0x12345678u) sink[0] = lds[0];
}

template <bool SCRATCH, bool SYNC>
static int run(bool cooperative, int wgs, unsigned* sink, const char* name) {
  const size_t lds = 120 * 1024;
  const void* fn = reinterpret_cast<const void*>(empty_kernel<SCRATCH, SYNC>);
  CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  std::vector<float> ms;
  for (int it = 0; it < 40; ++it) {
    int index = it;
    void* args[] = {&sink, &index};
    CHECK(hipEventRecord(e0));
    if (cooperative) CHECK(hipLaunchCooperativeKernel(fn, dim3(wgs), dim3(512), args, lds, 0));
    else hipLaunchKernelGGL((empty_kernel<SCRATCH, SYNC>), dim3(wgs), dim3(512), lds, 0, sink, index);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float t = 0.f;
    CHECK(hipEventElapsedTime(&t, e0, e1));
    if (it >= 10) ms.push_back(t);
  }
  std::sort(ms.begin(), ms.end());
  std::printf("%-44s median %6.2f us, fastest %6.2f us", name, ms[ms.size() / 2] * 1e3, ms[0] * 1e3);
  if (SYNC) {
    static unsigned long long h[kMaxWorkgroups][2];
    CHECK(hipMemcpyFromSymbol(h, HIP_SYMBOL(g_stamp), sizeof(h)));
    unsigned long long last_in = 0, last_out = 0;
    for (int i = 0; i < wgs; ++i) {
      last_in = std::max(last_in, h[i][0]);
      last_out = std::max(last_out, h[i][1]);
    }
    std::printf("; grid sync: last workgroup in -> last one out %.1f us", (double)(last_out - last_in) / 100.0);
  }
  std::printf("\n");
  return 0;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int wgs = std::min(prop.multiProcessorCount, kMaxWorkgroups);
  unsigned* sink = nullptr;
  CHECK(hipMalloc(&sink, (size_t)wgs * 64 * 4 + 64));
  std::printf("%d workgroups of 512 threads, 120 KB of LDS each\n", wgs);
  if (run<false, false>(false, wgs, sink, "plain launch") ||
      run<true, false>(false, wgs, sink, "plain launch, scratch memory in use") ||
      run<false, false>(true, wgs, sink, "cooperative launch") ||
      run<false, true>(true, wgs, sink, "cooperative launch, one grid-wide sync"))
    return 1;
  CHECK(hipFree(sink));
  return 0;
}
