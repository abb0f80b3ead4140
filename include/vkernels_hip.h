/*
 * vkernels_hip.h — C ABI of libvkernels_hip.so, the MI355X (gfx950) build of
 * the fused MXFP4 Mixture-of-Experts path.
 *
 * The entry points keep the names, argument order and conventions of the
 * reference's device ABI (src/c/vkernels/capi/hip_capi.hpp) so that a caller
 * that binds the reference's library — the ctypes loader in
 * src/python/vkernels/vllm_experts.py:388-459, the harness in
 * tests/python/test_mxfp4_serving_parity.py:200-225 — binds this one
 * unchanged.  Entry points marked "additive" have no counterpart in the
 * reference and follow the same conventions.
 *
 * Conventions (src/c/vkernels/capi/hip_capi.hpp:24-40):
 *   - every pointer is caller-owned DEVICE memory unless stated otherwise;
 *   - launchers enqueue work on `stream` (NULL = the default stream) and
 *     return at once: no allocation, no synchronisation, safe to capture in a
 *     HIP graph;
 *   - launchers that return void report launch errors through
 *     hipGetLastError() after the caller synchronises;
 *   - launchers that return int validate their arguments on the host and
 *     return VK_OK or a VK_ERROR_* code; the message of the last failure on
 *     the calling thread is available from vk_last_error().
 */
#ifndef VKERNELS_HIP_H_
#define VKERNELS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  Replaces src/c/vkernels/capi/capi.hpp:41-47.  (vkernels_cpu.h declares
 * the same codes under the same guard.) */
#ifndef VKERNELS_STATUS_CODES_
#define VKERNELS_STATUS_CODES_
enum {
  VK_OK = 0,
  VK_ERROR_INVALID_ARGUMENT = 1,
  VK_ERROR_OUT_OF_RANGE = 2,
  VK_ERROR_UNSUPPORTED = 3,
  VK_ERROR_INTERNAL = 4
};
#endif

/* Activation tags.  Replaces MoEActivation,
 * src/c/vkernels/kernels/moe_fused.hpp:47-50. */
enum { VK_MOE_SWIGLU = 0, VK_MOE_SITU = 1 };

/* Library version string.  Replaces src/c/vkernels/capi/capi.hpp:54. */
const char* vk_version(void);

/* 0: this build has no CUDA path.  Replaces capi.hpp:57. */
int vk_has_cuda(void);

/* Thread-local message / code of the most recent failing call on this
 * thread ("" / VK_OK if none).  Replaces capi.hpp:60-63. */
const char* vk_last_error(void);
int vk_last_error_code(void);

/* Set the thread-local error state.  Replaces capi.hpp:68. */
void vk_set_last_error(int code, const char* message);

/* Release memory returned by the library (nothing in this ABI allocates; kept
 * so that bindings that import the symbol still load).  Replaces capi.hpp:71. */
void vk_free(void* p);

/* Upper bound on the padded row count EM for (M, top_k, block_size,
 * num_experts): (ceil(M*top_k/block_size) + num_experts) * block_size; the
 * size to give sorted_ids (and /block_size for expert_ids).  Host arithmetic
 * only.  Replaces vk_moe_align_block_size_max_em,
 * src/c/vkernels/capi/capi.hpp:537-539 (capi_moe.cpp:110-117). */
size_t vk_moe_align_block_size_max_em(int32_t M, int32_t top_k,
                                      int32_t block_size, int32_t num_experts);

/*
 * Fused MXFP4 MoE layer: gate/up grouped GEMM with inline E2M1 x ue8m0
 * dequantisation, bias, SwiGLU or SiTU epilogue (one bf16 rounding) into
 * act_scratch, then the down grouped GEMM, bias, routing weight and
 * accumulation into out.
 * Replaces vk_hip_fused_moe_mxfp4, src/c/vkernels/capi/hip_capi.hpp:99-108
 * (src/c/vkernels/capi/hip_capi.cpp:40-57).
 *
 *   A           [M, hidden]            bf16 bit patterns
 *   w13         [E, 2*ispp, hidden/2]  packed E2M1, gate rows [0,ispp), up
 *                                      rows [ispp,2*ispp), low nibble = even k
 *   w13_scale   [E, 2*ispp, hidden/32] ue8m0
 *   w2          [E, hidden, ispp/2]    packed E2M1
 *   w2_scale    [E, hidden, ispp/32]   ue8m0
 *   topk_ids    [M, top_k]             routing table (not read; kept for ABI)
 *   topk_w      [M, top_k]             routing weights, read as topk_w[flat]
 *   act_scratch [EM, ispp]             bf16, indexed by sorted row; rows of
 *                                      padding are left untouched
 *   out         [M, hidden]            fp32; the caller zero-initialises it
 *                                      and the call ACCUMULATES into it
 *   sorted_ids  [EM]                   flat index token*top_k+sel per sorted
 *                                      row; entries >= M*top_k are padding
 *   expert_ids  [EM/block_size]        expert of each block; < 0 = skip
 *   EM          padded row count the two arrays were built for (may be the
 *               host's upper bound; padding blocks/rows are skipped)
 *   block_size  the alignment sorted_ids/expert_ids were built with; any
 *               positive multiple of 16
 *   hidden, ispp multiples of 64
 *   b13         [E, 2*ispp] fp32 or null; b2 [E, hidden] fp32 or null; aligned
 *               like any float array (4 bytes), as in the reference
 *   activation  0 = SwiGLU (g, u clamped by swiglu_limit when it is > 0),
 *               1 = SiTU with beta, linear_beta
 */
void vk_hip_fused_moe_mxfp4(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale,
    const int32_t* topk_ids, const float* topk_w,
    uint16_t* act_scratch, float* out,
    int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids,
    int EM, float swiglu_limit,
    int activation, float beta, float linear_beta,
    const float* b13, const float* b2, int block_size, void* stream);

/*
 * Additive: vk_hip_fused_moe_mxfp4 with a caller-owned device workspace, for
 * callers that can provide one (the library itself allocates nothing).  With
 * at least vk_hip_fused_moe_mxfp4_workspace_bytes(M, hidden, ispp, top_k, EM)
 * bytes, 16-byte aligned, the prefill-sized path splits the bf16 rows into their
 * FP8 terms once per call instead of once per workgroup, and its second stage
 * stores its rows (fp32, [EM, hidden], the bulk of the workspace) for a last pass
 * that sums each token's rows in selection order, instead of one atomic add per
 * row and column; results agree to fp32 rounding.
 * A null or short workspace is vk_hip_fused_moe_mxfp4 exactly.  The contents
 * of the workspace are unspecified after the call; calls that share one
 * must be ordered on a stream.  No counterpart in the reference, whose Python
 * binding owns the scratch of its fused call the same way
 * (src/python/vkernels/vllm_experts.py:160-214).
 */
size_t vk_hip_fused_moe_mxfp4_workspace_bytes(int M, int hidden, int ispp, int top_k, int EM);

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
    void* workspace, size_t workspace_bytes, void* stream);

/*
 * Additive: vk_hip_fused_moe_mxfp4_ws with flags.  VK_HIP_MOE_OVERWRITE_OUT:
 * `out` need not be initialised; the call clears it while its first stage runs
 * and the result is the layer alone (saves the caller's clearing launch, which
 * costs as much as 4 % of a decode-sized call).  Whenever M and EM are
 * positive and the arguments valid, that is: a call that returns early leaves
 * `out` as it is.  flags = 0 is vk_hip_fused_moe_mxfp4_ws exactly.  No
 * counterpart in the reference.
 */
#define VK_HIP_MOE_OVERWRITE_OUT 1u

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
    void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/*
 * Additive: weights prepacked at load time for the prefill-sized kernels, in
 * the spirit of the reference's `kmajor` layout option
 * (src/c/vkernels/kernels/moe_fused.hpp:315-343): a caller that keeps a second
 * copy of the expert weights in the layout the matrix cores consume gets the
 * FP4-rate path for batches of more than 512 routed rows.
 *
 * vk_hip_moe_prepack_weights rewrites [num_experts, rows, K/2] packed E2M1
 * codes and [num_experts, rows, K/32] ue8m0 scales (stage 0: w13 with rows =
 * 2*ispp, gate rows first, K = hidden; stage 1: w2 with rows = hidden, K =
 * ispp) into `packed`, vk_hip_moe_prepack_bytes(...) bytes of 16-byte aligned
 * device memory: per expert, per unit of 128 weight rows (stage 0: 64 gate
 * rows and the 64 up rows of the same columns), per K step of 128, the unit's
 * 8 operand tiles of 64 lanes x 16 bytes in lane order (codes moved onto the
 * OCP FP4 code points), then 8 scale bytes per lane (decremented by one); then
 * one flag byte per unit marking units whose weights hold an inf/NaN code or a
 * scale byte outside [64, 190]: such a unit is computed by the exact path, and
 * its blocks hold the codes and scale bytes as they are in w / w_scale (the move
 * onto the OCP points would merge the inf / NaN codes with others).  Returns VK_OK
 * or a VK_ERROR_* code.
 *
 * vk_hip_fused_moe_mxfp4_prepacked is vk_hip_fused_moe_mxfp4_ex with the two
 * packed buffers (NULL, NULL = vk_hip_fused_moe_mxfp4_ex exactly) and the
 * number of experts in the weight tensors.  With the packed buffers every kernel
 * family reads the prepacked form: decode-sized calls run decode kernels that
 * stream it (faster than the raw form's: the scale bytes come with the codes
 * and nothing is checked or moved in the loop), and both exact paths read it as
 * well.  The raw tensors are therefore optional: w13, w13_scale, w2 and w2_scale
 * may all be NULL (one copy of the weights), provided the call is one the decode
 * kernels take (vk_hip_moe_decode_max_rows routed rows: 512, or a number of rows per
 * expert in blocks of 16 or 32; rows of any width) or the workspace is given; otherwise
 * the call is
 * refused with VK_ERROR_INVALID_ARGUMENT in the error state.  On the packed path of
 * prefill-sized calls the bf16
 * activations are multiplied as a sum of FP6 (E2M3) terms per block of 32 along K,
 * each term with a block scale of its own: three terms (exact unless an element
 * lies more than 2^-13 below its block's largest) in the first stage, whose
 * error passes through the activation function and the second GEMM, and two
 * terms (error at most 2^-10 of the block's largest per element) in the second
 * (three there too when ispp < 1024: short sums average less, and such layers
 * are small): 5e-4 relative L2 of the layer against the reference's bf16
 * arithmetic.
 * VK_HIP_MOE_SPLIT3 selects three terms in both stages (7e-5; 12 % more
 * matrix-core work), VK_HIP_MOE_SPLIT2 two in both (1.4e-3, worst element 1e-2
 * of the RMS on the benchmark layers and up to 1.9e-2 on randomised small ones
 * with sums of 128 products: inside the reference's tolerance of 5e-3 / 2e-2,
 * with little margin; 25 % less work.  Its first-stage error is relative to the pre-activations,
 * so a swiglu_limit far below their spread magnifies it: with a limit of 1.5
 * against pre-activations of +-50 it measured 4.5e-3 / 5.7e-2, outside the
 * tolerance, where the default stays at 7e-5 / 1e-3).
 * The workspace size is vk_hip_fused_moe_mxfp4_workspace_bytes(...), as for _ws.
 */
#define VK_HIP_MOE_SPLIT2 2u
#define VK_HIP_MOE_SPLIT3 8u
/* VK_HIP_MOE_W4A4: the W4A4 mode of the reference's orchestration ops
 * (src/c/vkernels/kernels/moe_aux.hpp:1-25): both stages quantise their
 * activations (A, then act) to MXFP4 exactly as mxfp4_moe_quant does and multiply
 * FP4 by FP4, one matrix-core pass per product.  The layer then equals the
 * reference's layer applied to the dequantised quantised activations. */
#define VK_HIP_MOE_W4A4 4u

size_t vk_hip_moe_prepack_bytes(int32_t num_experts, int32_t rows, int32_t K, int32_t stage);

int vk_hip_moe_prepack_weights(const uint8_t* w, const uint8_t* w_scale, int32_t num_experts,
                               int32_t rows, int32_t K, int32_t stage, void* packed,
                               size_t packed_bytes, void* stream);

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
    const void* w13_packed, const void* w2_packed, int num_experts, void* stream);

/*
 * Additive: per-device set-up that the launchers otherwise do on their first
 * call (the dynamic-LDS limits of the GEMM kernels, the device address of the
 * library's scratch array, the tuning store of the launch shapes).  Call it
 * once per device, with that device current, before capturing a HIP graph
 * that contains the entry points of this library.  Returns VK_OK or a
 * VK_ERROR_* code.  No counterpart in the reference, whose launcher reads its
 * one environment knob on first use (src/c/vkernels/kernels/moe_fused.hip:1520-1523).
 */
int vk_hip_init(void);

/*
 * Additive: the launch-shape heuristics of the MoE kernels, as the reference
 * keeps its GEMM ones (candidate table
 * src/c/vkernels/kernels/common/heuristics.hpp:20-61; tuning store
 * src/c/vkernels/core/tuning.hpp:11-25, consulted before the compiled-in rules).
 *
 * vk_hip_moe_default_block_size: the alignment block the kernels like best for
 * M tokens routed to top_k experts each (what to pass to
 * vk_hip_moe_align_block_size and on to the layer).  Any multiple of 16 works.
 * vk_hip_moe_default_block_size_ex: the same for a caller that gives the prepacked
 * weights of num_local_experts experts of a hidden x ispp layer: what decides between
 * the decode kernels and the tile kernels (blocks of 128) is then rows per expert.  16 up
 * to 256 routed rows (where the first stage's kernel can align for itself); beyond, 32 up
 * to 28 rows per expert: the decode kernel of that form takes a block of 32 rows in one
 * pass over the expert's weights.  (A caller who passes blocks of 16 beyond 512 routed
 * rows still gets the decode kernels up to 9 rows per expert.)
 * vk_hip_moe_decode_max_rows: the routed rows (M * top_k) up to which a call in blocks of
 * block_size runs the decode kernels (num_local_experts: of a caller that gives the
 * prepacked weights, else 0; blocks of 32 are the decode kernels' only on that form).
 *
 * A launch shape is four ints {variant, wavefronts, tiles, depth}: variant 2 =
 * the decode kernel (one workgroup per compute unit, a run's rows resident in
 * LDS), 3 = the same with the K steps of a unit shared between wavefronts (a
 * single token), 4 = the decode kernel of the prepacked form that holds the rows a
 * chunk of K at a time (rows of any K; blocks of 16 or of 32 rows, the 32 rows of a
 * block in one pass over the expert's weights), 0 = the tile kernels; wavefronts per
 * workgroup; 16-row weight tiles per wavefront; K steps in flight per wavefront.
 * vk_hip_moe_tile_candidates writes up to `capacity` shapes that stage 0
 * (gate/up) or 1 (down) can be launched at and returns how many there are.
 * vk_hip_moe_tile_query writes the shape a call of this problem size would be
 * planned with and returns 1 when it comes from the tuning store, 0 from the
 * compiled-in rules (a launcher still falls back to the tile kernels where a
 * shape does not fit the device's LDS); stage 2 / 3 ask for stage 0 / 1 of a call
 * that gives the prepacked weights, whose decode kernels have rules of their own
 * (the store's records are shared), stage 4 / 5 of such a call in blocks of 32 rows.
 * vk_hip_moe_tile_set puts a record for (stage, K, ncols, bucket of n_flat)
 * into the process's store (shape null: removes it); VK_ERROR_INVALID_ARGUMENT
 * for a shape that is not a candidate.  vk_hip_moe_tuning_load reads
 * <dir>/moe_fused.gfx950.tune (dir null: $VKERNELS_TUNING_CACHE, default
 * ~/.cache/vkernels/tuning, "off" = none; also read on first use) and returns
 * the number of records taken.  vk_hip_moe_tuning_dump writes the store as the
 * text of such a file into buf (at most capacity bytes, always terminated) and
 * returns the length the whole text needs.
 */
int vk_hip_moe_default_block_size(int M, int top_k);
int vk_hip_moe_default_block_size_ex(int M, int top_k, int num_local_experts, int hidden, int ispp);
int vk_hip_moe_decode_max_rows(int num_local_experts, int block_size);
int vk_hip_moe_tile_candidates(int stage, int* shapes, int capacity);
int vk_hip_moe_tile_query(int stage, int K, int ncols, int n_flat, int* shape);
int vk_hip_moe_tile_set(int stage, int K, int ncols, int n_flat, const int* shape);
int vk_hip_moe_tuning_load(const char* dir);
size_t vk_hip_moe_tuning_dump(char* buf, size_t capacity);

/*
 * Additive: vk_hip_fused_moe_mxfp4_ex for callers that cannot allocate device
 * memory and have no workspace to lend: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  The workspace is an array of
 * vk_hip_static_scratch_bytes() (64 MiB) that the library itself holds in
 * device memory on every GPU it runs on, from the loading of its code until
 * the process ends; the call allocates nothing, frees nothing and does not
 * synchronise.  Arguments and results are those of vk_hip_fused_moe_mxfp4_ex
 * given a workspace of the size it asks for (the same kernels run).
 *
 * Returns VK_OK, VK_ERROR_INVALID_ARGUMENT for a contract violation, or
 * VK_ERROR_OUT_OF_RANGE when vk_hip_fused_moe_mxfp4_workspace_bytes(M, hidden,
 * ispp, top_k, EM) exceeds the array (nothing is launched; use
 * vk_hip_fused_moe_mxfp4_ws with a workspace of the caller's).
 *
 * All calls on one GPU share that GPU's array: calls that may overlap on one
 * GPU (different streams, different threads) race and must be ordered by the
 * caller.  The array keeps the last call's contents; nothing in it has to start
 * at zero, because every byte a call reads it has written before.  The array's
 * device address is looked up on the first call on a device (or by
 * vk_hip_init), which may load the library's code onto that device.
 */
size_t vk_hip_static_scratch_bytes(void);

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
    unsigned flags, void* stream);

/*
 * Additive: the two stages of vk_hip_fused_moe_mxfp4 as separate launches,
 * for callers that place work between them (a tensor-parallel all-reduce, a
 * profiler's events).  Device counterparts of the reference's stage split,
 * src/c/vkernels/kernels/moe_fused.hpp:103-125, with the activation fused
 * into the first stage and the combine into the second; calling one after the
 * other on a stream is exactly vk_hip_fused_moe_mxfp4.  Arguments as there.
 */
void vk_hip_moe_gateup_mxfp4(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    uint16_t* act_scratch, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    float swiglu_limit, int activation, float beta, float linear_beta,
    const float* b13, int block_size, void* stream);

void vk_hip_moe_down_mxfp4(
    const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
    const float* topk_w, float* out, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    const float* b2, int block_size, void* stream);

/*
 * Additive: vk_hip_moe_gateup_mxfp4 with the prepacked gate/up weights (NULL = raw
 * weights only).  With them, decode-sized calls run the decode kernels that read the
 * prepacked form, as the fused call does, and w13 / w13_scale may then be NULL; larger
 * calls run the raw-weight kernels and need the raw tensors.
 */
void vk_hip_moe_gateup_mxfp4_ex(
    const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
    uint16_t* act_scratch, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    float swiglu_limit, int activation, float beta, float linear_beta,
    const float* b13, int block_size, const void* w13_packed, int num_experts, void* stream);

/*
 * Additive: vk_hip_moe_down_mxfp4 with the optional arguments of the fused
 * entry points: a caller-owned workspace (size as for vk_hip_fused_moe_mxfp4_ws),
 * flags (VK_HIP_MOE_OVERWRITE_OUT, VK_HIP_MOE_SPLIT2) and the prepacked down
 * weights (NULL = raw weights only; with them w2 / w2_scale may be NULL when the
 * call is decode-sized or the workspace is given).  It runs the second stage exactly as the
 * fused call does for the same arguments, so a tensor-parallel caller can sum
 * `act` contributions between the stages and a test can feed the second stage
 * chosen `act` rows.  Device counterpart of moe_down_cpu + moe_combine_cpu,
 * src/c/vkernels/kernels/moe_fused.hpp:259-283.
 */
void vk_hip_moe_down_mxfp4_ex(
    const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
    const float* topk_w, float* out, int M, int hidden, int ispp, int top_k,
    const int32_t* sorted_ids, const int32_t* expert_ids, int EM,
    const float* b2, int block_size, void* workspace, size_t workspace_bytes, unsigned flags,
    const void* w2_packed, int num_experts, void* stream);

/*
 * Additive, for tests: bf16 rows [rows, K] -> the split rows the prefill-sized
 * kernels multiply: per row `terms` (2 or 3) planes of Kp = K rounded up to 128
 * bytes; a plane is Kp/32 blocks of 32 bytes: the 32 FP6 (E2M3) codes of the
 * term (code i at bit 6 i), the term's scale byte (the largest exponent field
 * of what the terms before it left of the block, less 2, at least 64), 7 zero
 * bytes.  row_flags[r] = 1 when a block of the row is outside the range of the
 * split (inf/NaN, first scale byte outside [64 + 4 (terms-1), 190]).  `split`
 * holds rows * terms * Kp bytes.
 */
int vk_hip_split_rows_fp6(const uint16_t* x, int32_t rows, int32_t K, int32_t terms, void* split,
                          uint8_t* row_flags, void* stream);

/*
 * Additive: device counterparts of the reference's MXFP4 MoE orchestration ops
 * (CPU ABI src/c/vkernels/capi/capi.hpp:470-503, semantics
 * src/c/vkernels/kernels/moe_aux.hpp:40-158), bit-identical to them:
 *   vk_hip_mxfp4_moe_quant         A [M, hidden] bf16 -> packed [M, hidden/2] E2M1
 *                                  codes (low nibble = even k) and scales
 *                                  [M, hidden/32] ue8m0 (0xFF = zero group)
 *   vk_hip_mxfp4_moe_sorted_quant  the same for row sorted_ids[r] / top_k of A per
 *                                  sorted row r; padding rows (id outside
 *                                  [0, M*top_k)) give zero codes and 0xFF scales
 *   vk_hip_mxfp4_moe_scatter_reduce out[token, :] += partial[r, :] * topk_w[r] for
 *                                  every routed sorted row r, in ascending r (gather
 *                                  form: no atomics; workspace: M*top_k int32)
 *   vk_hip_mxfp4_moe_sort          A_sorted[r, :] = A[sorted_ids[r] / top_k, :], bf16 rows
 *                                  of `hidden` values, a padding row zeroed
 *                                  (moe_aux.hpp:75, moe_aux.cpp:209-234)
 *   vk_hip_mxfp4_moe_sort_scales   the same for rows of n_groups ue8m0 bytes
 *                                  (moe_aux.hpp:90, moe_aux.cpp:236-260)
 *   vk_hip_mxfp4_moe_scatter_reduce_q  the routed combine of a quantised partial:
 *                                  partial_q [EM, width/2] E2M1 codes, partial_s
 *                                  [EM, width/32] ue8m0 (0xFF = zero), dequantised
 *                                  inline; the same order and roundings as the
 *                                  reference (moe_aux.hpp:174, moe_aux.cpp:288-321);
 *                                  out accumulates; workspace: M*top_k int32
 * group_size must be 32.  Return VK_OK or a VK_ERROR_* code.
 */
int vk_hip_mxfp4_moe_sort(const uint16_t* A, const int32_t* sorted_ids, uint16_t* A_sorted, int32_t M,
                          int32_t hidden, int32_t top_k, int32_t EM, void* stream);
int vk_hip_mxfp4_moe_sort_scales(const uint8_t* scales, const int32_t* sorted_ids, uint8_t* scales_sorted,
                                 int32_t M, int32_t n_groups, int32_t top_k, int32_t EM, void* stream);
int vk_hip_mxfp4_moe_scatter_reduce_q(const uint8_t* partial_q, const uint8_t* partial_s,
                                      const float* topk_w, const int32_t* sorted_ids, float* out,
                                      int32_t M, int32_t width, int32_t top_k, int32_t EM,
                                      int32_t group_size, void* workspace, size_t workspace_bytes,
                                      void* stream);
int vk_hip_mxfp4_moe_quant(const uint16_t* A, uint8_t* packed, uint8_t* scales, int32_t M,
                           int32_t hidden, int32_t group_size, void* stream);
int vk_hip_mxfp4_moe_sorted_quant(const uint16_t* A, const int32_t* sorted_ids, uint8_t* packed,
                                  uint8_t* scales, int32_t M, int32_t hidden, int32_t group_size,
                                  int32_t top_k, int32_t EM, void* stream);
int vk_hip_mxfp4_moe_scatter_reduce(const float* partial, const float* topk_w,
                                    const int32_t* sorted_ids, float* out, int32_t M, int32_t width,
                                    int32_t top_k, int32_t EM, void* workspace,
                                    size_t workspace_bytes, void* stream);

/*
 * Additive: the layer as four stages with an explicit boundary between the
 * linear GEMMs and the elementwise epilogues, for tensor-parallel callers that
 * sum (all-reduce) the fp32 pre-activations of their K slices between them.
 * Device counterparts of the reference's stage split
 * (src/c/vkernels/kernels/moe_fused.hpp:103-125; HIP declarations :259-283
 * moe_gateup_preact / moe_act_epilogue / moe_down_preact / moe_combine, which the
 * reference's C ABI does not export), with block_size as one more argument
 * (the reference's are fixed at 16) and the stream last:
 *
 *   vk_hip_moe_gateup_preact  gate_up[r, 0:ispp] = A[token(r), k_base : k_base +
 *       hidden_k] . w13[e, 0:ispp]^T, gate_up[r, ispp:2*ispp] likewise with the up
 *       rows, fp32 [EM, 2*ispp]; A rows are `hidden` wide, w13 / w13_scale are the
 *       rank's shard [E, 2*ispp, hidden_k/2] / [E, 2*ispp, hidden_k/32]
 *   (caller: all-reduce gate_up)
 *   vk_hip_moe_act_epilogue   act[r, :] = activation(gate_up[r] + b13[e]), bf16
 *       [EM, ispp]
 *   vk_hip_moe_down_preact    partial[r, :] = act[r, k_base : k_base + ispp_k] .
 *       w2[e]^T, fp32 [EM, hidden]; act rows are `ispp` wide, w2 / w2_scale the
 *       shard [E, hidden, ispp_k/2] / [E, hidden, ispp_k/32]
 *   (caller: all-reduce partial)
 *   vk_hip_moe_combine        out[token, :] += (partial[r, :] + b2[e, :]) *
 *       topk_w_sorted[r] over the token's sorted rows in ascending r: the sum
 *       the reference forms, bit for bit (gather form, no atomics; workspace:
 *       M*top_k int32 of device memory); topk_w_sorted is [EM], the routing
 *       weight of every sorted row (out accumulates: zero it first)
 *
 * With k_base = 0 and the full K the four calls compute what
 * vk_hip_fused_moe_mxfp4 computes.  Only routed rows (sorted id in
 * [0, M*top_k), block with an expert) are written or read.  hidden_k and ispp_k
 * must be multiples of 64, k_base and the row widths multiples of 8 (rows are
 * read 16 bytes at a time).  The GEMM stages take raw weights and run the
 * decode kernels or the plain tile kernels.  Return VK_OK or a VK_ERROR_* code;
 * asynchronous on `stream`, no allocation.
 */
int vk_hip_moe_gateup_preact(const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
                             const int32_t* sorted_ids, const int32_t* expert_ids, float* gate_up,
                             int M, int hidden, int ispp, int top_k, int EM, int k_base, int hidden_k,
                             int block_size, void* stream);
int vk_hip_moe_act_epilogue(const float* gate_up, const float* b13, uint16_t* act,
                            const int32_t* sorted_ids, const int32_t* expert_ids, int M, int top_k,
                            int EM, int ispp, float swiglu_limit, int activation, float beta,
                            float linear_beta, int block_size, void* stream);
int vk_hip_moe_down_preact(const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
                           const int32_t* sorted_ids, const int32_t* expert_ids, float* partial, int M,
                           int ispp, int hidden, int top_k, int EM, int k_base, int ispp_k,
                           int block_size, void* stream);
int vk_hip_moe_combine(const float* partial, const float* b2, const float* topk_w_sorted,
                       const int32_t* sorted_ids, const int32_t* expert_ids, float* out, int M,
                       int hidden, int top_k, int EM, int block_size, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * Additive: the two GEMM stages of the split above on prepacked weights, so that a
 * tensor-parallel caller at prefill sizes runs the FP4-rate kernels as the fused call
 * does.  w13_packed / w2_packed: vk_hip_moe_prepack_weights of the rank's shard
 * (K = hidden_k / ispp_k) of num_experts experts.  With it the raw shard (w13 /
 * w13_scale, w2 / w2_scale) may be NULL: the exact paths read the packed form, and calls
 * of up to 512 routed rows run the decode kernels on it; a call that would need the raw
 * shard (no workspace at prefill sizes) is then refused with VK_ERROR_INVALID_ARGUMENT.  workspace:
 * vk_hip_moe_preact_workspace_bytes(stage, M, EM, k_dim) bytes, 16-byte aligned (the
 * split rows of the K slice).  flags: VK_HIP_MOE_SPLIT2 / _SPLIT3 as for the layer
 * (default: three FP6 terms per activation in the first stage, two in the second).
 * Calls of up to 512 routed rows, or without packed weights or workspace, run the decode
 * or raw-weight kernels as vk_hip_moe_gateup_preact / vk_hip_moe_down_preact do (the
 * decode kernels on the packed shard where it is given).  Same outputs, same rules:
 * routed rows only are written.
 */
size_t vk_hip_moe_preact_workspace_bytes(int stage, int M, int EM, int k_dim);
int vk_hip_moe_gateup_preact_prepacked(const uint16_t* A, const uint8_t* w13, const uint8_t* w13_scale,
                                       const void* w13_packed, int num_experts, const int32_t* sorted_ids,
                                       const int32_t* expert_ids, float* gate_up, int M, int hidden, int ispp,
                                       int top_k, int EM, int k_base, int hidden_k, int block_size,
                                       void* workspace, size_t workspace_bytes, unsigned flags, void* stream);
int vk_hip_moe_down_preact_prepacked(const uint16_t* act, const uint8_t* w2, const uint8_t* w2_scale,
                                     const void* w2_packed, int num_experts, const int32_t* sorted_ids,
                                     const int32_t* expert_ids, float* partial, int M, int ispp, int hidden,
                                     int top_k, int EM, int k_base, int ispp_k, int block_size, void* workspace,
                                     size_t workspace_bytes, unsigned flags, void* stream);

/*
 * On-device alignment of the routing table: stable bucket of the flat indices
 * by (local) expert, each expert padded to a multiple of block_size.
 * Replaces vk_hip_moe_align_block_size,
 * src/c/vkernels/capi/hip_capi.hpp:148-153 (hip_capi.cpp:66-95).
 *
 *   topk_ids    [M*top_k]       global expert ids; ids outside
 *                               [0,num_experts) are skipped
 *   expert_map  [num_experts]   global -> local (-1 = skip), or NULL (1:1)
 *   local_n                     experts on this rank (<= num_experts)
 *   max_EM                      host upper bound on EM, multiple of
 *                               block_size, > 0
 *   sorted_ids  [max_EM]        all entries written; padding = M*top_k
 *   expert_ids  [max_EM/block_size] all entries written; padding = -1
 *   out_EM      [1]             padded row count, at least one block
 *
 * Unlike the reference there is no M*top_k <= 1024 limit: any size runs on
 * the device and VK_ERROR_UNSUPPORTED is only returned for num_experts beyond
 * VK_HIP_ALIGN_MAX_EXPERTS.
 */
#define VK_HIP_ALIGN_MAX_EXPERTS 1024
int vk_hip_moe_align_block_size(
    const int32_t* topk_ids, const int32_t* expert_map,
    int32_t M, int32_t top_k, int32_t block_size,
    int32_t num_experts, int32_t local_n, int32_t max_EM,
    int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM,
    void* stream);

/*
 * Additive: softmax -> top-k -> renormalise router, one wavefront per token.
 * Follows the conventions of vk_hip_moe_align_block_size; the semantics are
 * those of src/python/vkernels/torch_ops/tokenspeed_amd/routing.py:59-157
 * without bias and with scaling factor 1: p = softmax(logits) in fp32, top_k
 * arg-max picks of p with ties to the lowest expert index, weights p[ids],
 * divided by their sum when renormalize != 0 (a zero sum divides by 1).
 *
 *   logits    [T, E]      fp32
 *   topk_ids  [T, top_k]  int32, selection order (descending probability)
 *   topk_w    [T, top_k]  fp32
 *   E <= VK_HIP_ROUTE_MAX_EXPERTS, 1 <= top_k <= min(E, VK_HIP_ROUTE_MAX_TOPK)
 */
#define VK_HIP_ROUTE_MAX_EXPERTS 1024
#define VK_HIP_ROUTE_MAX_TOPK 32
int vk_hip_moe_route_topk(const float* logits, int32_t T, int32_t E,
                          int32_t top_k, int32_t renormalize,
                          int32_t* topk_ids, float* topk_w, void* stream);

/*
 * Additive: vk_hip_moe_route_topk followed by vk_hip_moe_align_block_size,
 * with the same arguments, results and errors as the two calls
 * (num_experts = E).  No counterpart in the reference, whose router is a
 * Python function (routing.py:59-157) and whose alignment is a call of its
 * own (hip_capi.hpp:148-153).  For the smallest batches (T <= 16) the two
 * are ONE launch: every workgroup of the alignment routes the tokens itself,
 * a wavefront per token, and keeps the table in LDS.  A launch is a few
 * microseconds, of a step of forty to eighty there.  Larger batches run the
 * two kernels one after the other.
 */
int vk_hip_moe_route_align(const float* logits, int32_t T, int32_t E, int32_t top_k,
                           int32_t renormalize, const int32_t* expert_map, int32_t block_size,
                           int32_t local_n, int32_t max_EM, int32_t* topk_ids, float* topk_w,
                           int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM, void* stream);

/*
 * Additive: router, alignment and the layer behind one call -- what a serving loop
 * runs per MoE layer and step.  The arguments are those of vk_hip_moe_route_align
 * (logits [M, num_experts] in; topk_ids, topk_w, sorted_ids [max_EM], expert_ids
 * [max_EM / block_size], out_EM out, written as that call writes them) and of
 * vk_hip_fused_moe_mxfp4_prepacked (the layer's buffers, workspace, flags, optional
 * prepacked weights of num_local_experts experts; with them the raw tensors may be
 * NULL as for vk_hip_fused_moe_mxfp4_prepacked).  Up to 256 routed rows (M * top_k),
 * with num_experts <= 256, block_size 16 and shapes the decode kernels take, the
 * first stage's kernel aligns for itself: for a handful of tokens (M <= 16) it routes
 * as well and the step is two launches; beyond, the router has its launch and the step
 * is three.  Every other call runs vk_hip_moe_route_align and then the layer.  The
 * results are the same either way: the routing tables bit for bit, `out` as the layer
 * computes it.
 * M = 0 writes the alignment's sentinels and EM and leaves `out` as it is.  Returns
 * VK_OK or a VK_ERROR_* code; asynchronous on `stream`, no allocation.
 */
int vk_hip_moe_route_layer_mxfp4(
    const uint16_t* A, const float* logits, const uint8_t* w13, const uint8_t* w13_scale,
    const uint8_t* w2, const uint8_t* w2_scale, int32_t* topk_ids, float* topk_w,
    uint16_t* act_scratch, float* out, int M, int num_experts, int hidden, int ispp, int top_k,
    int renormalize, const int32_t* expert_map, int local_n, int block_size, int max_EM,
    int32_t* sorted_ids, int32_t* expert_ids, int32_t* out_EM, float swiglu_limit, int activation,
    float beta, float linear_beta, const float* b13, const float* b2, void* workspace,
    size_t workspace_bytes, unsigned flags, const void* w13_packed, const void* w2_packed,
    int num_local_experts, void* stream);

/*
 * Additive: dequantise an [N, K] tile of packed weights to bf16 with the
 * decode routines of the device library, written transposed as [K][N].
 * Device counterpart of dequant_weight_tile,
 * src/c/vkernels/kernels/moe_fused.hpp:217-235 (moe_fused.cpp:141-174), for
 * bit-exact checks of the weight decode.  group_size must be 32.
 * fast == 0 selects the integer-exact routine (every code, every scale byte):
 * the one the GEMM kernels' exact path multiplies by.  fast != 0 selects the
 * hardware conversion v_cvt_scalef32_pk_bf16_fp4 on the remapped codes (finite
 * codes, scale bytes 3..252); the GEMM kernels' fast paths do not call it: the
 * matrix cores decode the same remapped codes and decremented scale bytes
 * themselves, and those values are pinned by the one-hot tests of the second
 * stage instead.
 */
int vk_hip_dequant_weight_tile(const uint8_t* packed, const uint8_t* scale,
                               uint16_t* out_bf16, int32_t N, int32_t K,
                               int32_t group_size, int32_t stride_packed,
                               int32_t stride_scale_n, int32_t stride_scale_k,
                               int32_t fast, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VKERNELS_HIP_H_ */
