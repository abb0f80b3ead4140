// static_scratch.hip — the device memory the library itself holds.
//
// Callers that cannot allocate (code under HIP graph capture, serving loops
// and harnesses that forbid hipMalloc) reach the workspace path of the fused
// layer through vk_hip_fused_moe_mxfp4_static, whose workspace is the
// file-scope device array below instead of a caller's buffer.  The array is
// part of the code object: every GPU the library runs on holds its own copy,
// at its own address, from the time the code object is loaded until the
// process ends.
//
// In host code the array's name is a stand-in, not a device address, so the
// address is asked for once per device (hipGetSymbolAddress with that device
// current) and only that address is handed to launchers.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "vk_internal.hpp"

namespace vk {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_scratch_ptr[kMaxDevices];  // by device ordinal; null = not resolved yet

}  // namespace

size_t static_scratch_bytes() { return kStaticScratchBytes; }

// Address of the current device's copy of the array (resolved on the first
// call per device).  On failure returns null and leaves the HIP status in *err.
void* static_scratch_ptr(hipError_t* err) {
  int dev = 0;
  hipError_t st = hipGetDevice(&dev);
  if (st != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    if (err != nullptr) *err = st != hipSuccess ? st : hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    st = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (st != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();  // not left for the next caller to find
      if (err != nullptr) *err = st != hipSuccess ? st : hipErrorInvalidSymbol;
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  if (err != nullptr) *err = hipSuccess;
  return g_scratch_ptr[dev];
}

}  // namespace vk
