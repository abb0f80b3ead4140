// read_stream.hip — what a read-only kernel of the decode kernel's launch shape reaches on
// this device: one workgroup of 512 threads per compute unit, every wavefront a contiguous
// share of `MB` megabytes, 16 bytes per lane and load, D loads per lane in flight.  Rotates
// over buffers larger than the Infinity Cache, so every launch reads cold memory.  The
// time is between HIP events around the launch, as bench.py takes its kernel times.
//
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops vkernels_amd/microbench/read_stream.hip -o /tmp/read_stream
//   /tmp/read_stream [MB, default 284 = the weights of 32 experts of 2880 x 2880 gate/up]
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(call)                                                                        \
  do {                                                                                     \
    const hipError_t err_ = (call);                                                        \
    if (err_ != hipSuccess) {                                                              \
      std::fprintf(stderr, "%s line %d: %s\n", #call, __LINE__, hipGetErrorString(err_)); \
      return 1;                                                                            \
    }                                                                                      \
  } while (0)

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

template <int D>
__global__ __launch_bounds__(512) void read_kernel(const u32x4* src, size_t vec_per_wave, unsigned* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const u32x4* p = src + ((size_t)blockIdx.x * 8 + wave) * vec_per_wave + lane;
  const size_t loads = vec_per_wave / 64;  // per lane
  u32x4 st[D];
  unsigned acc = 0;
#pragma unroll
  for (int i = 0; i < D; ++i) st[i] = p[(size_t)i * 64];
  for (size_t k = D; k + D <= loads; k += D) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      acc ^= st[i][0] ^ st[i][1] ^ st[i][2] ^ st[i][3];
      st[i] = p[(k + i) * 64];
    }
  }
#pragma unroll
  for (int i = 0; i < D; ++i) acc ^= st[i][0] ^ st[i][3];
  if (acc == 0x12345678u) sink[0] = acc;  // never true for the fill below; keeps the loads
}

template <int D>
static int run(const char* buf, size_t bytes, int sets, int wgs, unsigned* sink) {
  const size_t vec_per_wave = bytes / 16 / ((size_t)wgs * 8) / 64 * 64;
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  std::vector<float> ms;
  for (int it = 0; it < 35; ++it) {
    const u32x4* src = reinterpret_cast<const u32x4*>(buf + (size_t)(it % sets) * bytes);
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(read_kernel<D>, dim3(wgs), dim3(512), 0, 0, src, vec_per_wave, sink);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float t = 0.f;
    CHECK(hipEventElapsedTime(&t, e0, e1));
    if (it >= 5) ms.push_back(t);
  }
  std::sort(ms.begin(), ms.end());
  const double read = (double)vec_per_wave * 16 * wgs * 8;
  const double med = ms[ms.size() / 2];
  std::printf("%2d loads in flight per lane: median %.1f us = %.0f GB/s (fastest %.1f us = %.0f GB/s)\n", D,
              med * 1e3, read / (med * 1e-3) / 1e9, ms[0] * 1e3, read / (ms[0] * 1e-3) / 1e9);
  return 0;
}

int main(int argc, char** argv) {
  const size_t bytes = (size_t)(argc > 1 ? std::atoi(argv[1]) : 284) << 20;
  const int sets = 5;
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int wgs = prop.multiProcessorCount;
  char* buf = nullptr;
  unsigned* sink = nullptr;
  CHECK(hipMalloc(&buf, bytes * sets));
  CHECK(hipMalloc(&sink, 64));
  CHECK(hipMemset(buf, 1, bytes * sets));
  std::printf("%zu MB per launch, %d workgroups of 512 threads\n", bytes >> 20, wgs);
  if (run<4>(buf, bytes, sets, wgs, sink) || run<8>(buf, bytes, sets, wgs, sink) ||
      run<16>(buf, bytes, sets, wgs, sink))
    return 1;
  CHECK(hipFree(buf));
  CHECK(hipFree(sink));
  return 0;
}
