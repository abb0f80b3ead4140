// hip_capi.cpp — the extern "C" surface of libvkernels_hip.so (declared in
// include/vkernels_hip.h).  Host-side argument checks and error state only;
// the kernels live in the moe_*.hip translation units.
#include "vkernels_hip.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <string>

#include "vk_internal.hpp"
#include "moe_tuning.hpp"

namespace {

thread_local std::string g_last_error;
thread_local int g_last_error_code = VK_OK;

int fail(int code, const char* message) {
  vk_set_last_error(code, message);
  return code;
}

}  // namespace

extern "C" {

const char* vk_version(void) { return "0.1.0"; }

int vk_has_cuda(void) { return 0; }

const char* vk_last_error(void) { return g_last_error.c_str(); }

int vk_last_error_code(void) { return g_last_error_code; }

void vk_set_last_error(int code, const char* message) {
  g_last_error_code = code;
  g_last_error = message != nullptr ? message : "";
}

void vk_free(void* p) { free(p); }

size_t vk_moe_align_block_size_max_em(int32_t M, int32_t top_k,
                                      int32_t block_size,
                                      int32_t num_experts) {
  if (block_size <= 0) return 0;
  const int32_t n = M * top_k;
  const int32_t max_em = ((n + block_size - 1) / block_size + num_experts) * block_size;
  return max_em > 0 ? static_cast<size_t>(max_em) : 0;
}

namespace {

// Shared contract check of the three layer entry points.  They return void
// like the reference's launcher; a violation is recorded for vk_last_error()
// and nothing is launched.
// A call that passes the prepacked weights in place of the raw tensors (all four null).
bool packed_weights_alone(const void* w13, const void* w13_scale, const void* w2, const void* w2_scale,
                          const void* w13_packed, const void* w2_packed) {
  return w13 == nullptr && w13_scale == nullptr && w2 == nullptr && w2_scale == nullptr &&
         w13_packed != nullptr && w2_packed != nullptr;
}
const char* const kPackedOnlyNeeds =
    "a call without the raw weights needs shapes the decode kernels take or, beyond them, the "
    "workspace of vk_hip_fused_moe_mxfp4_workspace_bytes (16-byte aligned)";

// packed_only: the call passes the prepacked weights in place of the raw tensors.
bool layer_args_ok(const char* who, bool need13, bool need2, const vk::FusedMoeArgs& a,
                   bool packed_only = false) {
  const char* why = nullptr;
  if (a.sorted_ids == nullptr || a.expert_ids == nullptr || a.act == nullptr)
    why = "buffers must not be null";
  else if (need13 && (a.A == nullptr || (!packed_only && (a.w13 == nullptr || a.w13_scale == nullptr))))
    why = "buffers must not be null";
  else if (need2 && ((!packed_only && (a.w2 == nullptr || a.w2_scale == nullptr)) || a.topk_w == nullptr ||
                     a.out == nullptr))
    why = "buffers must not be null";
  else if (a.hidden <= 0 || a.ispp <= 0 || a.hidden % 64 != 0 || a.ispp % 64 != 0)
    why = "hidden and ispp must be positive multiples of 64";
  else if (a.top_k <= 0)
    why = "top_k must be positive";
  else if (a.block_size <= 0 || a.block_size % 16 != 0 || a.EM % a.block_size != 0)
    why = "block_size must be a multiple of 16 and divide EM";
  else if (((reinterpret_cast<uintptr_t>(a.b13) | reinterpret_cast<uintptr_t>(a.b2)) & 3u) != 0)
    why = "b13 and b2 must be aligned like the floats they hold";
  if (why == nullptr) return true;
  vk_set_last_error(VK_ERROR_INVALID_ARGUMENT, (std::string(who) + ": " + why).c_str());
  return false;
}

}  // namespace

void vk_hip_fused_moe_mxfp4(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size, void* stream) {
  vk_hip_fused_moe_mxfp4_ws(A, w13, w13_scale, w2, w2_scale, topk_ids, topk_w, act_scratch, out,
                            M, hidden, ispp, top_k, sorted_ids, expert_ids, EM, swiglu_limit,
                            activation, beta, linear_beta, b13, b2, block_size, nullptr, 0, stream);
}

size_t vk_hip_fused_moe_mxfp4_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM) {
  return vk::fused_moe_workspace_bytes(M, hidden, ispp, top_k, EM);
}

void vk_hip_fused_moe_mxfp4_ws(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size,
    void* workspace, size_t workspace_bytes, void* stream) {
  vk_hip_fused_moe_mxfp4_ex(A, w13, w13_scale, w2, w2_scale, topk_ids, topk_w, act_scratch, out,
                            M, hidden, ispp, top_k, sorted_ids, expert_ids, EM, swiglu_limit,
                            activation, beta, linear_beta, b13, b2, block_size, workspace,
                            workspace_bytes, 0u, stream);
}

namespace {

// After the launches of an entry point: a launch the runtime refused is recorded for
// vk_last_error() (peeked, so hipGetLastError() still reports it to the caller as the
// conventions promise).  `before` is the runtime's error state peeked ahead of the
// launches: an error that an earlier, unrelated call left there stays that call's and is
// not reported as this one's.  True when this call's launches failed.
bool note_launch_error(const char* who, hipError_t before) {
  const hipError_t err = hipPeekAtLastError();
  if (err == hipSuccess || before != hipSuccess) return false;
  vk_set_last_error(VK_ERROR_INTERNAL,
                    (std::string(who) + ": launch failed: " + hipGetErrorString(err)).c_str());
  return true;
}

vk::FusedMoeArgs fused_args(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale, const float* topk_w,
    uint16_t* act_scratch, float* out, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM, float swiglu_limit,
    int activation, float beta, float linear_beta, const float* b13, const float* b2,
    int block_size, void* workspace, size_t workspace_bytes, unsigned flags) {
  vk::FusedMoeArgs a{};
  a.workspace = workspace; a.workspace_bytes = workspace_bytes; a.flags = flags;
  a.A = A; a.w13 = w13; a.w13_scale = w13_scale; a.w2 = w2; a.w2_scale = w2_scale;
  a.topk_w = topk_w; a.act = act_scratch; a.out = out;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.b13 = b13; a.b2 = b2;
  a.M = M; a.hidden = hidden; a.ispp = ispp; a.top_k = top_k; a.EM = EM;
  a.block_size = block_size; a.swiglu_limit = swiglu_limit; a.beta = beta;
  a.linear_beta = linear_beta; a.activation = activation;
  return a;
}

}  // namespace

void vk_hip_fused_moe_mxfp4_ex(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size,
    void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
  (void)topk_ids;
  if (M <= 0 || EM <= 0) return;  // nothing routed: out is left as it is
  const vk::FusedMoeArgs a =
      fused_args(A, w13, w13_scale, w2, w2_scale, topk_w, act_scratch, out, M, hidden, ispp,
                 top_k, sorted_ids, expert_ids, EM, swiglu_limit, activation, beta, linear_beta,
                 b13, b2, block_size, workspace, workspace_bytes, flags);
  if (!layer_args_ok("vk_hip_fused_moe_mxfp4", true, true, a)) return;
  const hipError_t before = hipPeekAtLastError();
  vk::launch_fused_moe(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_fused_moe_mxfp4", before);
}

void vk_hip_fused_moe_mxfp4_prepacked(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size,
    void* workspace, size_t workspace_bytes, unsigned flags,
    const void* w13_packed, const void* w2_packed, int num_experts, void* stream) {
  (void)topk_ids;
  if (M <= 0 || EM <= 0) return;  // nothing routed: out is left as it is
  vk::FusedMoeArgs a =
      fused_args(A, w13, w13_scale, w2, w2_scale, topk_w, act_scratch, out, M, hidden, ispp,
                 top_k, sorted_ids, expert_ids, EM, swiglu_limit, activation, beta, linear_beta,
                 b13, b2, block_size, workspace, workspace_bytes, flags);
  const bool packed_only = packed_weights_alone(w13, w13_scale, w2, w2_scale, w13_packed, w2_packed);
  if (!layer_args_ok("vk_hip_fused_moe_mxfp4_prepacked", true, true, a, packed_only)) return;
  if ((w13_packed == nullptr) != (w2_packed == nullptr) || (w13_packed != nullptr && num_experts <= 0)) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT,
                      "vk_hip_fused_moe_mxfp4_prepacked: both packed buffers (or neither) and a "
                      "positive num_experts are required");
    return;
  }
  a.w13_packed = static_cast<const uint8_t*>(w13_packed);
  a.w2_packed = static_cast<const uint8_t*>(w2_packed);
  a.num_experts = num_experts;
  if (packed_only && !vk::fused_moe_packed_only_ok(a)) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT, kPackedOnlyNeeds);
    return;
  }
  const hipError_t before = hipPeekAtLastError();
  vk::launch_fused_moe(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_fused_moe_mxfp4_prepacked", before);
}

void vk_hip_moe_down_mxfp4_ex(
    const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
    const float* topk_w, float* out, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    const float* b2, int block_size, void* workspace, size_t workspace_bytes, unsigned flags,
    const void* w2_packed, int num_experts, void* stream) {
  if (M <= 0 || EM <= 0) return;
  vk::FusedMoeArgs a{};
  a.w2 = w2; a.w2_scale = w2_scale; a.topk_w = topk_w;
  a.act = const_cast<uint16_t*>(act); a.out = out;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.b2 = b2;
  a.M = M; a.hidden = hidden; a.ispp = ispp; a.top_k = top_k; a.EM = EM;
  a.block_size = block_size;
  a.workspace = workspace; a.workspace_bytes = workspace_bytes; a.flags = flags;
  a.w2_packed = static_cast<const uint8_t*>(w2_packed);
  a.num_experts = num_experts;
  const bool packed_only = w2 == nullptr && w2_scale == nullptr && w2_packed != nullptr;
  if (!layer_args_ok("vk_hip_moe_down_mxfp4_ex", false, true, a, packed_only)) return;
  if (w2_packed != nullptr && num_experts <= 0) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT,
                      "vk_hip_moe_down_mxfp4_ex: num_experts must be positive with packed weights");
    return;
  }
  if (packed_only && !vk::moe_down_packed_only_ok(a)) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT, kPackedOnlyNeeds);
    return;
  }
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_down(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_moe_down_mxfp4_ex", before);
}

int vk_hip_split_rows_fp6(const uint16_t* x, int32_t rows, int32_t K, int32_t terms, void* split,
                          uint8_t* row_flags, void* stream) {
  if (rows < 0 || K <= 0 || K % 32 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "rows must be >= 0 and K a positive multiple of 32");
  if (terms != 2 && terms != 3)
    return fail(VK_ERROR_INVALID_ARGUMENT, "terms must be 2 or 3");
  if (rows == 0) return VK_OK;
  if (x == nullptr || split == nullptr || row_flags == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "x/split/row_flags must not be null");
  vk::launch_split_rows_fp6(x, rows, K, terms, static_cast<uint8_t*>(split), row_flags,
                            static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int32_t M,
                           int32_t hidden, int32_t group_size, void* stream) {
  if (group_size != 32) return fail(VK_ERROR_UNSUPPORTED, "group_size must be 32");
  if (M < 0 || hidden < 0 || hidden % 32 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "M and hidden must be non-negative, hidden a multiple of group_size");
  if (M == 0 || hidden == 0) return VK_OK;
  if (A == nullptr || packed == nullptr || scales == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "A/packed/scales must not be null");
  vk::launch_mxfp4_quant(A, nullptr, packed, scales, M, hidden, 1, M, static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_sorted_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed,
                                  uint8_t* scales, int32_t M, int32_t hidden, int32_t group_size,
                                  int32_t top_k, int32_t EM, void* stream) {
  if (group_size != 32) return fail(VK_ERROR_UNSUPPORTED, "group_size must be 32");
  if (M < 0 || hidden < 0 || EM < 0 || top_k <= 0 || hidden % 32 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "M, hidden, EM must be non-negative, top_k positive, hidden a multiple of group_size");
  if (EM == 0 || hidden == 0) return VK_OK;
  if (A == nullptr || sorted_ids == nullptr || packed == nullptr || scales == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "A/sorted_ids/packed/scales must not be null");
  vk::launch_mxfp4_quant(A, sorted_ids, packed, scales, EM, hidden, top_k, M * top_k,
                         static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int32_t M,
                          int32_t hidden, int32_t top_k, int32_t EM, void* stream) {
  if (M < 0 || hidden < 0 || top_k <= 0 || EM < 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "M, hidden, top_k, EM must be valid");
  if (EM == 0 || hidden == 0) return VK_OK;
  if (A == nullptr || sorted_ids == nullptr || A_sorted == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "A/sorted_ids/A_sorted must not be null");
  vk::launch_mxfp4_gather_rows(A, sorted_ids, A_sorted, sizeof(uint16_t) * (size_t)hidden, top_k, M * top_k,
                               EM, static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids, uint8_t* scales_sorted,
                                 int32_t M, int32_t n_groups, int32_t top_k, int32_t EM, void* stream) {
  if (M < 0 || n_groups < 0 || top_k <= 0 || EM < 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "M, n_groups, top_k, EM must be valid");
  if (EM == 0 || n_groups == 0) return VK_OK;
  if (scales == nullptr || sorted_ids == nullptr || scales_sorted == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "scales/sorted_ids/scales_sorted must not be null");
  vk::launch_mxfp4_gather_rows(scales, sorted_ids, scales_sorted, (size_t)n_groups, top_k, M * top_k, EM,
                               static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                      const float* topk_w, const int32_t* sorted_ids, float* out,
                                      int32_t M, int32_t width, int32_t top_k, int32_t EM,
                                      int32_t group_size, void* workspace, size_t workspace_bytes,
                                      void* stream) {
  if (group_size != 32) return fail(VK_ERROR_UNSUPPORTED, "group_size must be 32");
  if (M < 0 || width < 0 || EM < 0 || top_k <= 0 || width % 32 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "M, width, EM must be non-negative, top_k positive, width a multiple of group_size");
  if (M == 0 || width == 0 || EM == 0) return VK_OK;
  if (partial_q == nullptr || partial_s == nullptr || topk_w == nullptr || sorted_ids == nullptr ||
      out == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "partial_q/partial_s/topk_w/sorted_ids/out must not be null");
  if ((reinterpret_cast<uintptr_t>(partial_q) & 3u) != 0 || (reinterpret_cast<uintptr_t>(out) & 3u) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "partial_q and out must be 4-byte aligned");
  if (workspace == nullptr || workspace_bytes < sizeof(int32_t) * (size_t)M * (size_t)top_k ||
      (reinterpret_cast<uintptr_t>(workspace) & 3) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "workspace must hold M * top_k int32 values");
  vk::launch_mxfp4_scatter_reduce_q(partial_q, partial_s, topk_w, sorted_ids, out, M, width, top_k, EM,
                                    static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w,
                                    const int32_t* sorted_ids, float* out, int32_t M, int32_t width,
                                    int32_t top_k, int32_t EM, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  if (M < 0 || width < 0 || EM < 0 || top_k <= 0 || width % 4 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "M, width, EM must be non-negative, top_k positive, width a multiple of 4");
  if (M == 0 || width == 0 || EM == 0) return VK_OK;
  if (partial == nullptr || topk_w == nullptr || sorted_ids == nullptr || out == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "partial/topk_w/sorted_ids/out must not be null");
  if (((reinterpret_cast<uintptr_t>(partial) | reinterpret_cast<uintptr_t>(out)) & 3u) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "partial and out must be aligned like floats");
  if (workspace == nullptr || workspace_bytes < sizeof(int32_t) * (size_t)M * (size_t)top_k ||
      (reinterpret_cast<uintptr_t>(workspace) & 3) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "workspace must hold M * top_k int32 values");
  vk::launch_mxfp4_scatter_reduce(partial, topk_w, sorted_ids, out, M, width, top_k, EM,
                                  static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
  return VK_OK;
}

namespace {

// Shape rules the stage entry points share; null when they hold.
const char* stage_shape_error(int M, int width_a, int ncols, int top_k, int EM, int k_base, int k_dim,
                              int block_size) {
  if (M < 0 || EM < 0) return "M and EM must not be negative";
  if (width_a <= 0 || ncols <= 0 || ncols % 64 != 0 || width_a % 8 != 0)
    return "row widths must be positive, the output width a multiple of 64, the input width of 8";
  if (top_k <= 0) return "top_k must be positive";
  if (k_dim <= 0 || k_dim % 64 != 0 || k_base < 0 || k_base % 8 != 0 || k_base + k_dim > width_a)
    return "the K slice must be a multiple of 64 wide, start at a multiple of 8 and lie inside the rows";
  if (block_size <= 0 || block_size % 16 != 0 || EM % block_size != 0)
    return "block_size must be a multiple of 16 and divide EM";
  return nullptr;
}

int stage_launch_status(const char* who, hipError_t before) {
  return note_launch_error(who, before) ? VK_ERROR_INTERNAL : VK_OK;
}

}  // namespace

int vk_hip_moe_gateup_preact(const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
                             const int32_t* sorted_ids, const int32_t* expert_ids, float* gate_up,
                             int M, int hidden, int ispp, int top_k, int EM, int k_base, int hidden_k,
                             int block_size, void* stream) {
  if (const char* why = stage_shape_error(M, hidden, ispp, top_k, EM, k_base, hidden_k, block_size))
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string("vk_hip_moe_gateup_preact: ") + why).c_str());
  if (M == 0 || EM == 0) return VK_OK;
  if (A == nullptr || w13 == nullptr || w13_scale == nullptr || sorted_ids == nullptr ||
      expert_ids == nullptr || gate_up == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_gateup_preact: buffers must not be null");
  vk_set_last_error(VK_OK, "");
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_preact(0, A, w13, w13_scale, sorted_ids, expert_ids, gate_up, M, hidden, ispp, top_k, EM,
                        k_base, hidden_k, block_size, static_cast<hipStream_t>(stream));
  return stage_launch_status("vk_hip_moe_gateup_preact", before);
}

size_t vk_hip_moe_preact_workspace_bytes(int stage, int M, int EM, int k_dim) {
  return vk::mx_preact_workspace_bytes(stage, M, EM, k_dim);
}

namespace {

// The pre-activation GEMM of a stage, on prepacked weights where the call is one the
// FP4-rate kernels take (more routed rows than the decode kernels', a workspace), on the
// raw weights otherwise.
int preact_any(const char* who, int stage, const uint16_t* a, const uint8_t* w, const uint8_t* w_scale,
               const void* packed, int num_experts, const int32_t* sorted_ids, const int32_t* expert_ids,
               float* preact, int M, int width_a, int ncols, int top_k, int EM, int k_base, int k_dim,
               int block_size, void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
  if (const char* why = stage_shape_error(M, width_a, ncols, top_k, EM, k_base, k_dim, block_size))
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string(who) + ": " + why).c_str());
  if (M == 0 || EM == 0) return VK_OK;
  const bool raw_given = w != nullptr && w_scale != nullptr;
  if (a == nullptr || (!raw_given && (packed == nullptr || w != nullptr || w_scale != nullptr)) ||
      sorted_ids == nullptr || expert_ids == nullptr || preact == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string(who) + ": buffers must not be null").c_str());
  if (packed != nullptr && num_experts <= 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string(who) + ": num_experts must be positive with packed weights").c_str());
  vk_set_last_error(VK_OK, "");
  const hipError_t before = hipPeekAtLastError();
  const bool prefill_sized = (long long)M * top_k > vk::kMoeDecodeMaxRows;
  if (!(packed != nullptr && prefill_sized &&
        vk::launch_moe_preact_prepacked(stage, a, static_cast<const uint8_t*>(packed), w, w_scale, sorted_ids,
                                        expert_ids, preact, M, width_a, ncols, top_k, EM, k_base, k_dim,
                                        block_size, num_experts, workspace, workspace_bytes, flags,
                                        static_cast<hipStream_t>(stream))) &&
      !vk::launch_moe_preact(stage, a, w, w_scale, sorted_ids, expert_ids, preact, M, width_a, ncols, top_k, EM,
                             k_base, k_dim, block_size, static_cast<hipStream_t>(stream),
                             static_cast<const uint8_t*>(packed), num_experts))
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string(who) + ": " + kPackedOnlyNeeds).c_str());
  return stage_launch_status(who, before);
}

}  // namespace

int vk_hip_moe_gateup_preact_prepacked(const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
                                       const void* w13_packed, int num_experts, const int32_t* sorted_ids,
                                       const int32_t* expert_ids, float* gate_up, int M, int hidden, int ispp,
                                       int top_k, int EM, int k_base, int hidden_k, int block_size,
                                       void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
  return preact_any("vk_hip_moe_gateup_preact_prepacked", 0, A, w13, w13_scale, w13_packed, num_experts,
                    sorted_ids, expert_ids, gate_up, M, hidden, ispp, top_k, EM, k_base, hidden_k, block_size,
                    workspace, workspace_bytes, flags, stream);
}

int vk_hip_moe_down_preact_prepacked(const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
                                     const void* w2_packed, int num_experts, const int32_t* sorted_ids,
                                     const int32_t* expert_ids, float* partial, int M, int ispp, int hidden,
                                     int top_k, int EM, int k_base, int ispp_k, int block_size, void* workspace,
                                     size_t workspace_bytes, unsigned flags, void* stream) {
  return preact_any("vk_hip_moe_down_preact_prepacked", 1, act, w2, w2_scale, w2_packed, num_experts, sorted_ids,
                    expert_ids, partial, M, ispp, hidden, top_k, EM, k_base, ispp_k, block_size, workspace,
                    workspace_bytes, flags, stream);
}

int vk_hip_moe_act_epilogue(const float* gate_up, const float* b13, uint16_t* act,
                            const int32_t* sorted_ids, const int32_t* expert_ids, int M, int top_k,
                            int EM, int ispp, float swiglu_limit, int activation, float beta,
                            float linear_beta, int block_size, void* stream) {
  if (M < 0 || EM < 0 || top_k <= 0 || ispp <= 0 || ispp % 4 != 0 || block_size <= 0 ||
      EM % block_size != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "vk_hip_moe_act_epilogue: M, EM non-negative, top_k positive, ispp a positive multiple "
                "of 4, block_size a divisor of EM");
  if (activation != VK_MOE_SWIGLU && activation != VK_MOE_SITU)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_act_epilogue: unknown activation");
  if (M == 0 || EM == 0) return VK_OK;
  if (gate_up == nullptr || act == nullptr || sorted_ids == nullptr || expert_ids == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_act_epilogue: buffers must not be null");
  vk_set_last_error(VK_OK, "");
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_act_epilogue(gate_up, b13, act, sorted_ids, expert_ids, M, top_k, EM, ispp, block_size,
                              swiglu_limit, activation, beta, linear_beta,
                              static_cast<hipStream_t>(stream));
  return stage_launch_status("vk_hip_moe_act_epilogue", before);
}

int vk_hip_moe_down_preact(const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
                           const int32_t* sorted_ids, const int32_t* expert_ids, float* partial, int M,
                           int ispp, int hidden, int top_k, int EM, int k_base, int ispp_k,
                           int block_size, void* stream) {
  if (const char* why = stage_shape_error(M, ispp, hidden, top_k, EM, k_base, ispp_k, block_size))
    return fail(VK_ERROR_INVALID_ARGUMENT, (std::string("vk_hip_moe_down_preact: ") + why).c_str());
  if (M == 0 || EM == 0) return VK_OK;
  if (act == nullptr || w2 == nullptr || w2_scale == nullptr || sorted_ids == nullptr ||
      expert_ids == nullptr || partial == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_down_preact: buffers must not be null");
  vk_set_last_error(VK_OK, "");
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_preact(1, act, w2, w2_scale, sorted_ids, expert_ids, partial, M, ispp, hidden, top_k, EM,
                        k_base, ispp_k, block_size, static_cast<hipStream_t>(stream));
  return stage_launch_status("vk_hip_moe_down_preact", before);
}

int vk_hip_moe_combine(const float* partial, const float* b2, const float* topk_w_sorted,
                       const int32_t* sorted_ids, const int32_t* expert_ids, float* out, int M,
                       int hidden, int top_k, int EM, int block_size, void* workspace,
                       size_t workspace_bytes, void* stream) {
  if (M < 0 || EM < 0 || top_k <= 0 || hidden <= 0 || hidden % 4 != 0 || block_size <= 0 ||
      EM % block_size != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "vk_hip_moe_combine: M, EM non-negative, top_k positive, hidden a positive multiple of "
                "4, block_size a divisor of EM");
  if (M == 0 || EM == 0) return VK_OK;
  if (partial == nullptr || topk_w_sorted == nullptr || sorted_ids == nullptr || expert_ids == nullptr ||
      out == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_combine: buffers must not be null");
  if (((reinterpret_cast<uintptr_t>(partial) | reinterpret_cast<uintptr_t>(b2) |
        reinterpret_cast<uintptr_t>(out)) & 3u) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_combine: partial, b2 and out must be aligned like floats");
  if (workspace == nullptr || workspace_bytes < sizeof(int32_t) * (size_t)M * (size_t)top_k ||
      (reinterpret_cast<uintptr_t>(workspace) & 3) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_combine: workspace must hold M * top_k int32 values");
  vk_set_last_error(VK_OK, "");
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_combine_sorted(partial, b2, topk_w_sorted, sorted_ids, expert_ids, out, M, hidden, top_k,
                                EM, block_size, static_cast<int32_t*>(workspace),
                                static_cast<hipStream_t>(stream));
  return stage_launch_status("vk_hip_moe_combine", before);
}

size_t vk_hip_moe_prepack_bytes(int32_t num_experts, int32_t rows, int32_t K, int32_t stage) {
  if (stage != 0 && stage != 1) return 0;
  return vk::moe_prepack_bytes(num_experts, rows, K, stage);
}

int vk_hip_moe_prepack_weights(const uint8_t* w, const uint8_t* w_scale, int32_t num_experts,
                               int32_t rows, int32_t K, int32_t stage, void* packed,
                               size_t packed_bytes, void* stream) {
  if (stage != 0 && stage != 1)
    return fail(VK_ERROR_INVALID_ARGUMENT, "stage must be 0 (gate/up weights) or 1 (down weights)");
  if (num_experts <= 0 || rows <= 0 || K <= 0 || K % 64 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "num_experts and rows must be positive, K a positive multiple of 64");
  if (stage == 0 ? (rows % 128 != 0) : (rows % 64 != 0))
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "rows must be 2 * ispp with ispp a multiple of 64 (stage 0) or a multiple of 64 (stage 1)");
  if (w == nullptr || w_scale == nullptr || packed == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "w/w_scale/packed must not be null");
  if ((reinterpret_cast<uintptr_t>(packed) & 15) != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "w and packed must be 16-byte aligned");
  if (packed_bytes < vk::moe_prepack_bytes(num_experts, rows, K, stage))
    return fail(VK_ERROR_INVALID_ARGUMENT, "packed buffer smaller than vk_hip_moe_prepack_bytes()");
  vk::launch_moe_prepack(w, w_scale, num_experts, rows, K, stage, static_cast<uint8_t*>(packed),
                         static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_init(void) {
  hipError_t err = hipSuccess;
  if (vk::static_scratch_ptr(&err) == nullptr)
    return fail(VK_ERROR_INTERNAL,
                (std::string("vk_hip_init: the library's scratch array has no device address: ") +
                 hipGetErrorString(err)).c_str());
  if (!vk::prepare_moe_kernels())
    return fail(VK_ERROR_UNSUPPORTED, "vk_hip_init: the device refuses a kernel its LDS");
  return VK_OK;
}

int vk_hip_moe_default_block_size(int M, int top_k) {
  return vk::moe_default_block_size(M < 0 ? 0 : M, top_k < 0 ? 0 : top_k);
}

int vk_hip_moe_default_block_size_ex(int M, int top_k, int num_local_experts, int hidden, int ispp) {
  return vk::moe_default_block_size(M < 0 ? 0 : M, top_k < 0 ? 0 : top_k,
                                    num_local_experts < 0 ? 0 : num_local_experts, hidden, ispp);
}

int vk_hip_moe_decode_max_rows(int num_local_experts, int block_size) {
  if (block_size == 32) return num_local_experts > 0 ? vk::moe_decode_max_rows32(num_local_experts) : 0;
  if (block_size != 16) return vk::kMoeDecodeMaxRows;
  return vk::moe_decode_max_rows(num_local_experts < 0 ? 0 : num_local_experts);
}

int vk_hip_moe_tile_candidates(int stage, int* shapes, int capacity) {
  size_t n = 0;
  const vk::MoeTileCandidate* table = vk::moe_tile_candidates(&n);
  int count = 0;
  for (size_t i = 0; i < n; ++i) {
    if (table[i].stage != stage) continue;
    if (shapes != nullptr && count < capacity) {
      const vk::MoeTile& t = table[i].tile;
      const int row[4] = {t.variant, t.waves, t.nt, t.depth};
      for (int j = 0; j < 4; ++j) shapes[4 * count + j] = row[j];
    }
    ++count;
  }
  return count;
}

int vk_hip_moe_tile_query(int stage, int K, int ncols, int n_flat, int* shape) {
  vk::MoeTile t;
  // stage + 2: the stage on the prepacked form; stage + 4: ... with blocks of 32 rows
  const bool packed = stage >= 2 && stage <= 5;
  const int block_rows = stage >= 4 && stage <= 5 ? 32 : 16;
  if (packed) stage &= 1;
  const bool stored = vk::moe_tuning_find(stage, K, ncols, n_flat, &t);
  if (!stored) t = vk::pick_moe_tile(n_flat, K, ncols, stage, packed, 0, block_rows);
  if (shape != nullptr) {
    shape[0] = t.variant; shape[1] = t.waves; shape[2] = t.nt; shape[3] = t.depth;
  }
  return stored ? 1 : 0;
}

int vk_hip_moe_tile_set(int stage, int K, int ncols, int n_flat, const int* shape) {
  vk::MoeTile t{};
  if (shape != nullptr) t = vk::MoeTile{shape[0], shape[1], shape[2], shape[3]};
  if (!vk::moe_tuning_set(stage, K, ncols, n_flat, shape != nullptr ? &t : nullptr))
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "vk_hip_moe_tile_set: stage must be 0 or 1, sizes positive, and the shape one of "
                "vk_hip_moe_tile_candidates");
  return VK_OK;
}

int vk_hip_moe_tuning_load(const char* dir) { return vk::moe_tuning_load(dir); }

size_t vk_hip_moe_tuning_dump(char* buf, size_t capacity) {
  const std::string text = vk::moe_tuning_dump("vk_hip_moe_tuning_dump");
  if (buf != nullptr && capacity > 0) {
    const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
    memcpy(buf, text.data(), n);
    buf[n] = 0;
  }
  return text.size() + 1;
}

size_t vk_hip_static_scratch_bytes(void) { return vk::static_scratch_bytes(); }

int vk_hip_fused_moe_mxfp4_static(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size,
    unsigned flags, void* stream) {
  (void)topk_ids;
  if (M <= 0 || EM <= 0) return VK_OK;  // nothing routed: out is left as it is
  vk::FusedMoeArgs a =
      fused_args(A, w13, w13_scale, w2, w2_scale, topk_w, act_scratch, out, M, hidden, ispp,
                 top_k, sorted_ids, expert_ids, EM, swiglu_limit, activation, beta, linear_beta,
                 b13, b2, block_size, nullptr, 0, flags);
  if (!layer_args_ok("vk_hip_fused_moe_mxfp4_static", true, true, a))
    return VK_ERROR_INVALID_ARGUMENT;
  const size_t need = vk::fused_moe_workspace_bytes(M, hidden, ispp, top_k, EM);
  if (need > vk::static_scratch_bytes())
    return fail(VK_ERROR_OUT_OF_RANGE,
                ("vk_hip_fused_moe_mxfp4_static: this call needs " + std::to_string(need) +
                 " bytes of scratch, the library holds " +
                 std::to_string(vk::static_scratch_bytes()) +
                 "; use vk_hip_fused_moe_mxfp4_ws with a caller-owned workspace").c_str());
  hipError_t err = hipSuccess;
  a.workspace = vk::static_scratch_ptr(&err);
  if (a.workspace == nullptr)
    return fail(VK_ERROR_INTERNAL,
                (std::string("vk_hip_fused_moe_mxfp4_static: the library's scratch array has no "
                             "device address: ") + hipGetErrorString(err)).c_str());
  a.workspace_bytes = vk::static_scratch_bytes();
  const hipError_t before = hipPeekAtLastError();
  vk::launch_fused_moe(a, static_cast<hipStream_t>(stream));
  return note_launch_error("vk_hip_fused_moe_mxfp4_static", before) ? VK_ERROR_INTERNAL : VK_OK;
}

void vk_hip_moe_gateup_mxfp4(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    uint16_t* act_scratch, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    float swiglu_limit, int activation, float beta, float linear_beta,
    const float* b13, int block_size, void* stream) {
  if (M <= 0 || EM <= 0) return;
  vk::FusedMoeArgs a{};
  a.A = A; a.w13 = w13; a.w13_scale = w13_scale; a.act = act_scratch;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.b13 = b13;
  a.M = M; a.hidden = hidden; a.ispp = ispp; a.top_k = top_k; a.EM = EM;
  a.block_size = block_size; a.swiglu_limit = swiglu_limit; a.beta = beta;
  a.linear_beta = linear_beta; a.activation = activation;
  if (!layer_args_ok("vk_hip_moe_gateup_mxfp4", true, false, a)) return;
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_gateup(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_moe_gateup_mxfp4", before);
}

void vk_hip_moe_gateup_mxfp4_ex(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    uint16_t* act_scratch, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    float swiglu_limit, int activation, float beta, float linear_beta,
    const float* b13, int block_size, const void* w13_packed, int num_experts, void* stream) {
  if (M <= 0 || EM <= 0) return;
  vk::FusedMoeArgs a{};
  a.A = A; a.w13 = w13; a.w13_scale = w13_scale; a.act = act_scratch;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.b13 = b13;
  a.M = M; a.hidden = hidden; a.ispp = ispp; a.top_k = top_k; a.EM = EM;
  a.block_size = block_size; a.swiglu_limit = swiglu_limit; a.beta = beta;
  a.linear_beta = linear_beta; a.activation = activation;
  a.w13_packed = static_cast<const uint8_t*>(w13_packed);
  a.num_experts = num_experts;
  const bool packed_only = w13 == nullptr && w13_scale == nullptr && w13_packed != nullptr;
  if (!layer_args_ok("vk_hip_moe_gateup_mxfp4_ex", true, false, a, packed_only)) return;
  if (w13_packed != nullptr && num_experts <= 0) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT,
                      "vk_hip_moe_gateup_mxfp4_ex: num_experts must be positive with packed weights");
    return;
  }
  if (packed_only && !vk::moe_gateup_packed_only_ok(a)) {
    vk_set_last_error(VK_ERROR_INVALID_ARGUMENT,
                      "vk_hip_moe_gateup_mxfp4_ex: without the raw weights the first stage alone runs "
                      "at decode sizes only");
    return;
  }
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_gateup(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_moe_gateup_mxfp4_ex", before);
}

void vk_hip_moe_down_mxfp4(
    const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
    const float* topk_w, float* out, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    const float* b2, int block_size, void* stream) {
  if (M <= 0 || EM <= 0) return;
  vk::FusedMoeArgs a{};
  a.w2 = w2; a.w2_scale = w2_scale; a.topk_w = topk_w;
  a.act = const_cast<uint16_t*>(act); a.out = out;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.b2 = b2;
  a.M = M; a.hidden = hidden; a.ispp = ispp; a.top_k = top_k; a.EM = EM;
  a.block_size = block_size;
  if (!layer_args_ok("vk_hip_moe_down_mxfp4", false, true, a)) return;
  const hipError_t before = hipPeekAtLastError();
  vk::launch_moe_down(a, static_cast<hipStream_t>(stream));
  note_launch_error("vk_hip_moe_down_mxfp4", before);
}

int vk_hip_moe_align_block_size(
    const int32_t* topk_ids, const int32_t* expert_map,
    int32_t M, int32_t top_k, int32_t block_size,
    int32_t num_experts, int32_t local_n, int32_t max_EM,
    int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM,
    void* stream) {
  if (block_size <= 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "block_size must be positive");
  if (M < 0 || top_k < 0 || num_experts < 0 || local_n < 0 || max_EM < 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "sizes must be non-negative");
  if (max_EM == 0 || (max_EM % block_size) != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "max_EM must be a positive multiple of block_size");
  if (local_n > num_experts)
    return fail(VK_ERROR_INVALID_ARGUMENT, "local_n must not exceed num_experts");
  if (out_EM == nullptr || sorted_ids == nullptr || expert_ids == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "sorted_ids/expert_ids/out_EM must not be null");
  if (M > 0 && top_k > 0 && topk_ids == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "topk_ids must not be null");
  const long long n = static_cast<long long>(M) * static_cast<long long>(top_k);
  if (n > 0x7FFFFFFFll)
    return fail(VK_ERROR_OUT_OF_RANGE, "M*top_k does not fit in int32");
  if (local_n > VK_HIP_ALIGN_MAX_EXPERTS)
    return fail(VK_ERROR_UNSUPPORTED, "more local experts than VK_HIP_ALIGN_MAX_EXPERTS");
  vk::launch_align(topk_ids, expert_map, static_cast<int>(n), block_size, num_experts,
                   local_n, max_EM, sorted_ids, expert_ids, out_EM,
                   static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_moe_route_topk(const float* logits, int32_t T, int32_t E,
                          int32_t top_k, int32_t renormalize,
                          int32_t* topk_ids, float* topk_w, void* stream) {
  if (T < 0 || E <= 0 || top_k <= 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "T must be >= 0, E and top_k positive");
  if (top_k > E)
    return fail(VK_ERROR_INVALID_ARGUMENT, "top_k must not exceed E");
  if (E > VK_HIP_ROUTE_MAX_EXPERTS || top_k > VK_HIP_ROUTE_MAX_TOPK)
    return fail(VK_ERROR_UNSUPPORTED, "E or top_k beyond the router's limits");
  if (T == 0) return VK_OK;
  if (logits == nullptr || topk_ids == nullptr || topk_w == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "logits/topk_ids/topk_w must not be null");
  vk::launch_route_topk(logits, T, E, top_k, renormalize, topk_ids, topk_w,
                        static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_moe_route_align(const float* logits, int32_t T, int32_t E, int32_t top_k,
                           int32_t renormalize, const int32_t* expert_map, int32_t block_size,
                           int32_t local_n, int32_t max_EM, int32_t* topk_ids, float* topk_w,
                           int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM, void* stream) {
  // the shapes one launch does not take (and T = 0, where only the alignment has work:
  // the sentinels and out_EM) go through the two entry points, which check the rest
  if (T <= 0 || E <= 0 || top_k <= 0 || top_k > E || E > VK_HIP_ROUTE_MAX_EXPERTS ||
      top_k > VK_HIP_ROUTE_MAX_TOPK || block_size <= 0 || local_n < 0 || local_n > E ||
      max_EM <= 0 || max_EM % block_size != 0 || local_n > VK_HIP_ALIGN_MAX_EXPERTS ||
      logits == nullptr || topk_ids == nullptr || topk_w == nullptr || sorted_ids == nullptr ||
      expert_ids == nullptr || out_EM == nullptr || !vk::route_align_fits(T, E, top_k, local_n)) {
    const int rc = vk_hip_moe_route_topk(logits, T, E, top_k, renormalize, topk_ids, topk_w, stream);
    if (rc != VK_OK) return rc;
    return vk_hip_moe_align_block_size(topk_ids, expert_map, T, top_k, block_size, E, local_n, max_EM,
                                       sorted_ids, expert_ids, out_EM, stream);
  }
  vk::launch_route_align(logits, T, E, top_k, renormalize, expert_map, block_size, local_n, max_EM,
                         topk_ids, topk_w, sorted_ids, expert_ids, out_EM,
                         static_cast<hipStream_t>(stream));
  return VK_OK;
}

int vk_hip_moe_route_layer_mxfp4(
    const uint16_t* A, const float* logits, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale, int32_t* topk_ids, float* topk_w,
    uint16_t* act_scratch, float* out, int M, int num_experts, int hidden, int ispp, int top_k,
    int renormalize, const int32_t* expert_map, int local_n, int block_size, int max_EM,
    int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM, float swiglu_limit, int activation,
    float beta, float linear_beta, const float* b13, const float* b2, void* workspace,
    size_t workspace_bytes, unsigned flags, const void* w13_packed, const void* w2_packed,
    int num_local_experts, void* stream) {
  if (M <= 0) {  // nothing routed: the alignment still writes its sentinels and EM
    if (M < 0) return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_route_layer_mxfp4: M must be non-negative");
    return vk_hip_moe_align_block_size(topk_ids, expert_map, 0, top_k, block_size, num_experts, local_n,
                                       max_EM, sorted_ids, expert_ids, out_EM, stream);
  }
  vk::FusedMoeArgs a =
      fused_args(A, w13, w13_scale, w2, w2_scale, topk_w, act_scratch, out, M, hidden, ispp, top_k,
                 sorted_ids, expert_ids, max_EM, swiglu_limit, activation, beta, linear_beta, b13, b2,
                 block_size, workspace, workspace_bytes, flags);
  if (max_EM <= 0 || block_size <= 0 || max_EM % block_size != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_route_layer_mxfp4: block_size must divide max_EM");
  const bool packed_only = packed_weights_alone(w13, w13_scale, w2, w2_scale, w13_packed, w2_packed);
  if (!layer_args_ok("vk_hip_moe_route_layer_mxfp4", true, true, a, packed_only)) return VK_ERROR_INVALID_ARGUMENT;
  if (logits == nullptr || topk_ids == nullptr || out_EM == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "vk_hip_moe_route_layer_mxfp4: logits/topk_ids/out_EM must not be null");
  if ((w13_packed == nullptr) != (w2_packed == nullptr) || (w13_packed != nullptr && num_local_experts <= 0))
    return fail(VK_ERROR_INVALID_ARGUMENT,
                "vk_hip_moe_route_layer_mxfp4: both packed buffers (or neither) and a positive "
                "num_local_experts are required");
  a.w13_packed = static_cast<const uint8_t*>(w13_packed);
  a.w2_packed = static_cast<const uint8_t*>(w2_packed);
  a.num_experts = num_local_experts;
  if (packed_only && !vk::fused_moe_packed_only_ok(a)) return fail(VK_ERROR_INVALID_ARGUMENT, kPackedOnlyNeeds);
  if (num_experts > 0 && top_k <= num_experts && local_n >= 0 && local_n <= num_experts) {
    vk::RoutedArgs r{};
    r.logits = logits; r.expert_map = expert_map; r.topk_ids = topk_ids; r.topk_w = topk_w;
    r.sorted_ids = sorted_ids; r.expert_ids = expert_ids; r.out_EM = out_EM;
    r.num_experts = num_experts; r.local_n = local_n; r.renormalize = renormalize; r.max_EM = max_EM;
    const hipError_t before = hipPeekAtLastError();
    if (vk::launch_routed_moe(a, r, static_cast<hipStream_t>(stream)))
      return note_launch_error("vk_hip_moe_route_layer_mxfp4", before) ? VK_ERROR_INTERNAL : VK_OK;
  }
  // every other shape: router and alignment (one launch or two), then the layer
  const int rc = vk_hip_moe_route_align(logits, M, num_experts, top_k, renormalize, expert_map, block_size,
                                        local_n, max_EM, topk_ids, topk_w, sorted_ids, expert_ids, out_EM,
                                        stream);
  if (rc != VK_OK) return rc;
  const hipError_t before = hipPeekAtLastError();
  vk::launch_fused_moe(a, static_cast<hipStream_t>(stream));
  return note_launch_error("vk_hip_moe_route_layer_mxfp4", before) ? VK_ERROR_INTERNAL : VK_OK;
}

int vk_hip_dequant_weight_tile(const uint8_t* packed, const uint8_t* scale,
                               uint16_t* out_bf16, int32_t N, int32_t K,
                               int32_t group_size, int32_t stride_packed,
                               int32_t stride_scale_n, int32_t stride_scale_k,
                               int32_t fast, void* stream) {
  if (group_size != 32)
    return fail(VK_ERROR_UNSUPPORTED, "group_size must be 32");
  if (N < 0 || K < 0 || K % 32 != 0)
    return fail(VK_ERROR_INVALID_ARGUMENT, "N must be >= 0 and K a multiple of 32");
  if (N == 0 || K == 0) return VK_OK;
  if (packed == nullptr || scale == nullptr || out_bf16 == nullptr)
    return fail(VK_ERROR_INVALID_ARGUMENT, "packed/scale/out_bf16 must not be null");
  vk::launch_dequant_tile(packed, scale, out_bf16, N, K, stride_packed, stride_scale_n,
                          stride_scale_k, fast, static_cast<hipStream_t>(stream));
  return VK_OK;
}

}  // extern "C"
