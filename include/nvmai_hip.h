/*
 * nvmai_hip.h -- C ABI of the MI355X (gfx950) quantized mixture-of-experts hot path.
 *
 * Drop-in boundary for NVMAI's operator layer.  Each entry point replaces one
 * Swift operator wrapper of the reference (sources/NVMAI/Kernels/...) or one
 * function of its C target (sources/NVMAIKernelsC); the replaced interface is
 * cited above each declaration.  Conventions, mirroring the reference's
 * `encode(commandBuffer:...)` wrappers:
 *   - every pointer is a raw DEVICE pointer unless marked "host"; a Metal
 *     (buffer, byteOffset) pair becomes pointer + offset computed by the caller;
 *   - calls only enqueue work on `stream` (a hipStream_t) and never synchronise;
 *   - status is returned as int: 0 = ok, negative = nvmai_status; nothing aborts;
 *   - one nvmai_hip_ctx per stream; a ctx is not thread-safe.
 *   - workspace and HIP graphs: entry points take their intermediate buffers from a
 *     workspace the ctx owns.  It grows (hipMalloc) the first time a call needs more
 *     than any call before it; blocks it has outgrown stay allocated until
 *     nvmai_hip_ctx_destroy, so a captured graph stays valid whatever is called
 *     later.  A call that would have to grow while its stream is being captured
 *     returns NVMAI_ERR_SCRATCH and launches nothing: run the same call eagerly once,
 *     or nvmai_hip_ctx_reserve, before capturing.
 * Data formats (reference file:line):
 *   - weights: affine group-64 codes, 4 bit (two per byte, element 2k in the low
 *     nibble of byte k) or 8 bit, plus one BF16 scale and one BF16 bias per group
 *     (nvmai_kernels.h:10-21, Quantization.swift:32-38).  Code rows must be
 *     16-byte aligned.
 *   - activations: 16-bit, BF16 or FP16 chosen at ctx creation.
 *   - routing weights, softmax probabilities, KV scale/bias: FP16.
 */
#ifndef NVMAI_HIP_H
#define NVMAI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nvmai_hip_ctx nvmai_hip_ctx;
typedef void* nvmai_stream;   /* hipStream_t */

typedef enum {
    NVMAI_OK = 0,
    NVMAI_ERR_INVALID_ARG = -1,   /* shape/size contract violated (reference: precondition) */
    NVMAI_ERR_UNSUPPORTED = -2,   /* e.g. weight bits not in {4,8} (SharedExpertError.unsupportedWeightBits) */
    NVMAI_ERR_ALIGNMENT = -3,     /* a pointer or stride is not 16-byte aligned */
    NVMAI_ERR_SCRATCH = -4,       /* caller scratch too small (SharedExpertError.scratchTooSmall) */
    NVMAI_ERR_HIP = -5,           /* a HIP runtime call failed */
    NVMAI_ERR_NO_DEVICE = -6
} nvmai_status;

enum { NVMAI_ACT_BF16 = 0, NVMAI_ACT_FP16 = 1 };

/* Rows in "router format": kind 4 / 8 = affine codes with BF16 scale/bias per
 * group of 64; kind 16 = dense BF16 (scales/biases unused); kind 0 = absent. */
typedef struct {
    const void* weights;
    const uint16_t* scales;
    const uint16_t* biases;
    int32_t kind;
} nvmai_rows;

/* Byte offsets of the nine tensors of one expert blob.
 * Replaces MoEExpertOffsets (MoE.swift:5-29) == ExpertOffsets (moe.metal:141-151). */
typedef struct {
    uint32_t gate_w, gate_s, gate_b, up_w, up_s, up_b, down_w, down_s, down_b;
} nvmai_expert_offsets;

/* Replaces MetalContext (MetalContext.swift) for this path: binds a device,
 * fixes the activation type, owns the small persistent scratch the reference's
 * wrappers own (router logits MoE.swift:130-139, split-KV partials
 * Attention.swift:117-126, sampler stages LogitOutput.swift:244-258). */
int nvmai_hip_ctx_create(int device, int act_dtype, nvmai_hip_ctx** out);
void nvmai_hip_ctx_destroy(nvmai_hip_ctx* ctx);
/* Grow the ctx workspace to at least `bytes` now (the counterpart of the wrappers' scratch
 * buffers allocated in init, Attention.swift:117-126, LogitOutput.swift:244-258), so that no
 * later call has to; nvmai_hip_ctx_workspace_bytes reports the current size. */
int nvmai_hip_ctx_reserve(nvmai_hip_ctx* ctx, size_t bytes);
size_t nvmai_hip_ctx_workspace_bytes(const nvmai_hip_ctx* ctx);
const char* nvmai_hip_status_string(int status);

/* Per-kernel timing, the counterpart of the reference's NVMAI_KERNEL_STATS roles
 * (RealForwardRunner.swift:1129-1188): while enabled, each tagged kernel launch is
 * bracketed by events on its stream.  profile_read waits for the recorded events,
 * returns the summed milliseconds and launch count of one tag and leaves the
 * records in place; profile_enable(…, 1) clears them. */
enum {
    NVMAI_PROF_ROUTER = 0, NVMAI_PROF_SELECT = 1, NVMAI_PROF_GROUP = 2, NVMAI_PROF_PHASE1 = 3,
    NVMAI_PROF_PHASE2 = 4, NVMAI_PROF_COMBINE = 5, NVMAI_PROF_KV_QUANT = 6, NVMAI_PROF_ATTN_PARTIAL = 7,
    NVMAI_PROF_ATTN_COMBINE = 8, NVMAI_PROF_SOFTMAX = 9, NVMAI_PROF_SAMPLE = 10,
    NVMAI_PROF_PREFILL_GROUP = 11, NVMAI_PROF_PREFILL_GEMM1 = 12, NVMAI_PROF_PREFILL_GEMM2 = 13,
    NVMAI_PROF_PREFILL_COMBINE = 14, NVMAI_PROF_TAGS = 16
};
int nvmai_hip_profile_enable(nvmai_hip_ctx* ctx, int on);
int nvmai_hip_profile_read(nvmai_hip_ctx* ctx, int tag, double* total_ms, uint32_t* launches);

/* No counterpart in the reference: a measuring stick for the roofline fractions.  Reads `bytes` (a multiple of 16,
 * 16-byte aligned) of device memory and does nothing else -- what a kernel that only streams reaches on this
 * device, to set beside the rate of the library's own streaming kernels in the same run.  `sink` (may be NULL) is
 * never written in practice; it only keeps the loads alive. */
int nvmai_hip_read_probe(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* data, uint64_t bytes, uint32_t* sink);

/* CPUExpertFFN.Offsets(d:f:) (CPUExpertFFN.swift:42-59) for `bits` in {4,8}.
 * Host-only arithmetic; *stride_bytes receives the blob size. */
int nvmai_expert_offsets_for(uint32_t d, uint32_t f, uint32_t bits,
                             nvmai_expert_offsets* out, uint64_t* stride_bytes);

/* Quantization.quantizeInt4Affine / quantizeInt8Affine (Quantization.swift:50-102,
 * 135-177) for a [rows, n] matrix on the device.  w is FP32 (w_is_bf16 = 0) or
 * BF16.  Codes, scale bits and bias bits equal the reference's bit for bit. */
int nvmai_hip_quantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* w,
                              int w_is_bf16, uint32_t rows, uint32_t n, uint32_t bits,
                              uint8_t* packed, uint16_t* scales, uint16_t* biases);

/* Quantization.dequantizeInt4Affine / Int8 (Quantization.swift:104-119, 179-191):
 * codes_out (one byte per code) and/or values_out (activations) may be NULL. */
int nvmai_hip_dequantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* packed,
                                const uint16_t* scales, const uint16_t* biases, uint64_t count,
                                uint32_t bits, uint8_t* codes_out, void* values_out);

/* DequantInt4GEMV.encode / DequantInt8GEMV.encode / AffineQuantGEMV.encode
 * (DequantInt4GEMV.swift:66-110, DequantInt8GEMV.swift:50-86, AffineQuant.swift:58)
 * and, with y_f32 != NULL, nvmai_int4_affine_gemv (nvmai_kernels.h:22-28):
 * y[t, :] = W x[t, :] for n_tokens inputs.  y (activations) or y_f32 may be NULL.
 * More than four inputs against a matrix of 32,768 rows or more (more than 32 inputs: 1024 rows), 16-bit outputs only and 16-byte
 * aligned operands: runs as nvmai_hip_affine_qmm (the matrix is read once for all inputs).
 * bits == 16: `weights` holds dense BF16 rows [m, n] (scales and biases unused, may be NULL; the
 * BF16 LM head): a BF16 context only, n a multiple of 64 and at most 4096, any number of inputs
 * (the matrix is read once per 16 of them). */
int nvmai_hip_affine_gemv(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                          const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                          const void* x, uint32_t x_stride, uint32_t n_tokens, uint32_t m,
                          uint32_t n, void* y, float* y_f32, uint32_t y_stride);

/* nvmai_int4_affine_gemv (nvmai_kernels.h:22-28, int4_affine_gemv.c:28-135) with the
 * reference's own signature: HOST pointers, 4-bit codes, BF16 scale/bias, fp32 x, out written
 * (not accumulated), n a multiple of 64.  The operands are copied to device 0, the GEMV runs
 * there and the call returns when `out` is complete.  It allocates and synchronises on every
 * call: it exists so that CPUExpertFFN's call sites keep linking; the fast path is
 * nvmai_hip_affine_gemv on resident weights.  A failure is reported on stderr and fills `out`
 * with NaN. */
void nvmai_int4_affine_gemv(const uint8_t* weights, const uint16_t* scales, const uint16_t* biases,
                            const float* x, size_t rows, size_t n, float* out);

/* MoE.encodeRouter (MoE.swift:151-213) and PrefillRouter.encodeBlock
 * (PrefillRouter.swift:41-95): logits for n_tokens rows of `hidden`, top-k by
 * (score desc, index asc), softmax over the selected, times per_expert_scale.
 * eff_scale / per_expert_scale are optional BF16 arrays (NULL = 1.0).
 * out_idx [n_tokens, top_k] u32, out_w [n_tokens, top_k] FP16;
 * logits_out optional FP32 [n_tokens, num_experts]. */
int nvmai_hip_moe_router_topk(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_rows* router,
                              const void* hidden, uint32_t hidden_stride, uint32_t n_tokens,
                              const uint16_t* eff_scale, const uint16_t* per_expert_scale,
                              uint32_t num_experts, uint32_t d, uint32_t top_k,
                              uint32_t* out_idx, uint16_t* out_w, float* logits_out);

/* MoE.encodeRoutedPersistentPhase1U16Load (MoE.swift:295-339; kernels
 * moe.metal:642-683, 812-834): acts[slot, :] = silu(gate_slot x) * (up_slot x)
 * for the top_k blobs in `blobs` (host array of top_k device pointers, the
 * reference's RoutedBlobs argument buffer).  acts is caller-owned FP32
 * [top_k, f]. */
int nvmai_hip_moe_phase1_gate_up_act(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                     const void* const* blobs, const nvmai_expert_offsets* off,
                                     uint32_t bits, const void* x, float* acts, uint32_t d,
                                     uint32_t f, uint32_t top_k);

/* MoE.encodeRoutedPersistentPhase1SubsetU16Load (MoE.swift:341-392; kernels
 * moe.metal:685-727, 836-861): same over active_slots[0..active_count) (device
 * array); slots >= top_k are skipped, rows of other slots stay untouched. */
int nvmai_hip_moe_phase1_gate_up_act_subset(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                            const void* const* blobs,
                                            const nvmai_expert_offsets* off, uint32_t bits,
                                            const void* x, float* acts, uint32_t d, uint32_t f,
                                            uint32_t top_k, const uint32_t* active_slots,
                                            uint32_t active_count);

/* MoE.encodeRoutedPersistentPhase2Reduce (MoE.swift:394-440; kernels
 * moe.metal:769-810, 863-892): y[d] = residual[d] + sum over slots in slot order
 * of w[slot] * (down_slot[d, :] . acts[slot, :]).  routing_w is FP16 [top_k];
 * residual (activations, may be NULL = 0) and y are [d]. */
int nvmai_hip_moe_phase2_down_reduce(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                     const void* const* blobs, const nvmai_expert_offsets* off,
                                     uint32_t bits, const float* acts, const uint16_t* routing_w,
                                     const void* residual, void* y, uint32_t d, uint32_t f,
                                     uint32_t top_k);

/* SharedExpertRuntime.encode (SharedExpertInt4.swift:100-153) plus the scalar
 * gate of RealForwardRunner.swift:3884-3900:
 * y[t, :] = sigmoid(gate . x[t]) * down(silu(gate_proj x[t]) * (up_proj x[t])).
 * The three projections live in one blob addressed by `off`; shared_gate may be
 * NULL or kind 0 (no gate). */
int nvmai_hip_shared_expert(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* blob,
                            const nvmai_expert_offsets* off, uint32_t bits,
                            const nvmai_rows* shared_gate, const void* x, uint32_t x_stride,
                            uint32_t n_tokens, void* y, uint32_t y_stride, uint32_t d, uint32_t f);

/* One MoE layer for a decode batch with every expert resident in HBM
 * (RealForwardRunner.swift:1900-1920 router, :3866-3912 shared expert, :3914-4297
 * routed experts, minus the two host round trips and the SSD streaming):
 * y[t] = sigmoid(g.x[t]) * ffn_shared(x[t]) + sum_slot w[t,slot] * ffn_{idx[t,slot]}(x[t]).
 * Each distinct routed expert is read once per call (with one or two tokens, where the step is
 * a chain of launches rather than bytes, each token reads its own experts and the call is three
 * launches instead of five). */
typedef struct {
    uint32_t d, f, num_experts, top_k, bits;
    nvmai_rows router;
    const void* experts_base;        /* expert e at experts_base + e * expert_stride */
    uint64_t expert_stride;
    nvmai_expert_offsets offsets;
    const void* shared_blob;         /* NULL = no shared expert */
    nvmai_rows shared_gate;          /* kind 0 = ungated */
    const uint16_t* eff_scale;       /* optional BF16 [d] */
    const uint16_t* per_expert_scale;/* optional BF16 [num_experts] */
} nvmai_moe_layer;

/* out_idx [n_tokens, top_k] u32 and out_w FP16 may be NULL; stats (optional,
 * device u32[2]) receives {work entries, distinct routed experts}. */
int nvmai_hip_moe_decode_layer(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* layer,
                               const void* x, uint32_t x_stride, uint32_t n_tokens, void* y,
                               uint32_t y_stride, uint32_t* out_idx, uint16_t* out_w,
                               uint32_t* stats);

/* The MoE block of a layer together with the residual add and the RMSNorm that open it
 * (RealForwardRunner's encodeResidualAdd, utility.metal:95-104, RMSNorm.encodeBF16W,
 * rmsnorm.metal:64-110, then the MoE calls of nvmai_hip_moe_decode_layer):
 *   hidden_out = round(hidden + delta)      (delta NULL: hidden_out = hidden)
 *   normed     = rmsnorm(hidden_out) * norm_weight
 *   y          = MoE(normed)
 * with the bits of nvmai_hip_residual_add_rmsnorm followed by nvmai_hip_moe_decode_layer.  Below 64
 * tokens, with 16-byte aligned rows and hidden_out, normed and hidden three different buffers, the
 * router launch norms its input itself (one launch fewer per layer); otherwise the steps run one
 * after the other.  normed is written for the caller too (the reference keeps it for the
 * shared-expert and the next projections). */
int nvmai_hip_moe_decode_layer_prenorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* layer,
                                       const void* hidden, uint32_t hidden_stride, const void* delta,
                                       uint32_t delta_stride, const uint16_t* norm_weight, float eps,
                                       void* hidden_out, uint32_t hidden_out_stride, void* normed,
                                       uint32_t normed_stride, uint32_t n_tokens, void* y, uint32_t y_stride,
                                       uint32_t* out_idx, uint16_t* out_w, uint32_t* stats);

/* The same with the residual add that closes the layer and the RMSNorm that opens the next one
 * (RealForwardRunner.swift:1857-1920: encodeResidualAdd after the MoE block, then the next layer's
 * RMSNorm.encodeBF16W):
 *   hidden_out  = round(hidden + delta);  normed = rmsnorm(hidden_out) * norm_weight;  y = MoE(normed)
 *   hidden_out  = round(hidden_out + y)
 *   next_normed = rmsnorm(hidden_out) * next_norm_weight
 * with the bits of nvmai_hip_moe_decode_layer_prenorm followed by nvmai_hip_residual_add_rmsnorm.
 * From five tokens on (the work-list path) the last two lines ride in the block's combine launch,
 * one block per token; otherwise they are the residual-add-norm kernel after the block.  hidden_out
 * ends as the residual stream after the layer; next_normed must be a buffer of its own. */
int nvmai_hip_moe_decode_layer_norms(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_moe_layer* layer,
                                     const void* hidden, uint32_t hidden_stride, const void* delta,
                                     uint32_t delta_stride, const uint16_t* norm_weight, float eps,
                                     void* hidden_out, uint32_t hidden_out_stride, void* normed,
                                     uint32_t normed_stride, uint32_t n_tokens, void* y, uint32_t y_stride,
                                     uint32_t* out_idx, uint16_t* out_w, uint32_t* stats,
                                     const uint16_t* next_norm_weight, void* next_normed,
                                     uint32_t next_normed_stride);

/* nvmai_hip_moe_decode_layer for callers that cannot allocate.  It has no counterpart in the
 * reference: it is for code under HIP graph capture, tight serving loops and harnesses that
 * forbid hipMalloc.  Same arguments, same results bit for bit, but the step's intermediate
 * buffers (router logits, work list, activations, partial sums) live in a static device array
 * of nvmai_hip_moe_decode_layer_noalloc_scratch_bytes() = 4 MiB inside the library, whose
 * device address the ctx looked up when it was created: the call allocates nothing, frees
 * nothing and records no memset, only kernel launches.  A step that needs more than the array
 * holds (the production shape fits 32 tokens: hidden 2048, intermediate 512, 256 experts,
 * top-8, shared expert) returns NVMAI_ERR_SCRATCH and launches nothing.  Every call on one
 * GPU shares that GPU's array and finds the previous call's contents in it (each call writes
 * what it reads, nothing has to be cleared): calls that overlap on one GPU, from different
 * streams or contexts, race.  The ctx's device must be the current device (each GPU has its own
 * copy of the array at its own address): otherwise NVMAI_ERR_INVALID_ARG. */
int nvmai_hip_moe_decode_layer_noalloc(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                       const nvmai_moe_layer* layer, const void* x, uint32_t x_stride,
                                       uint32_t n_tokens, void* y, uint32_t y_stride, uint32_t* out_idx,
                                       uint16_t* out_w, uint32_t* stats);
size_t nvmai_hip_moe_decode_layer_noalloc_scratch_bytes(void);


/* ---- prefill: permutation by expert and grouped expert GEMM ------------------------------- */

/* PrefillTokenExpertPair (PrefillRouter.swift:5-28 == prefill.metal:220-225): 16 bytes;
 * weight_bits holds the FP16 routing weight in its low 16 bits. */
typedef struct { uint32_t token, expert, rank, weight_bits; } nvmai_prefill_pair;
/* PrefillMoEGroup / PrefillMoETile (PrefillMoEGrouping.swift:4-29). */
typedef struct { uint32_t expert, pair_start, pair_count; } nvmai_prefill_group;
typedef struct { uint32_t group_start, group_count, pair_start, pair_count; } nvmai_prefill_tile;

/* PrefillMoEGroupingError (PrefillMoEGrouping.swift:52-89), numbered in declaration order. */
typedef enum {
    NVMAI_GROUPING_OK = 0, NVMAI_GROUPING_INVALID_QUERY_COUNT = 1, NVMAI_GROUPING_INVALID_TOP_K = 2,
    NVMAI_GROUPING_INVALID_NUM_EXPERTS = 3, NVMAI_GROUPING_INVALID_TILE_EXPERT_COUNT = 4,
    NVMAI_GROUPING_PAIR_COUNT_MISMATCH = 5, NVMAI_GROUPING_TOKEN_OUT_OF_RANGE = 6,
    NVMAI_GROUPING_RANK_OUT_OF_RANGE = 7, NVMAI_GROUPING_EXPERT_OUT_OF_RANGE = 8,
    NVMAI_GROUPING_DUPLICATE_TOKEN_RANK = 9, NVMAI_GROUPING_SORT_KEY_COUNT_MISMATCH = 10
} nvmai_grouping_error;

/* PrefillMoEGroupedRoutes (PrefillMoEGrouping.swift:31-50) as caller-owned DEVICE arrays:
 * sorted_pairs [n_pairs]; expert_offsets / expert_counts [num_experts] (offset 0xFFFFFFFF for
 * an expert without pairs); groups and tiles [num_experts] of which info[0] / info[1] are
 * filled.  info is u32[8]: {groups, tiles, nvmai_grouping_error found on the device (6..9 or
 * 0), index of the first failing pair, largest group, 0, 0, 0}. */
typedef struct {
    nvmai_prefill_pair* sorted_pairs;
    uint32_t* expert_offsets;
    uint32_t* expert_counts;
    nvmai_prefill_group* groups;
    nvmai_prefill_tile* tiles;
    uint32_t* info;
} nvmai_prefill_grouping;

/* The argument checks groupTokenExpertPairs makes before it looks at a pair
 * (PrefillMoEGrouping.swift:99-119); host only.  Returns a nvmai_grouping_error. */
int nvmai_prefill_grouping_check(int64_t n_pairs, int64_t query_count, int64_t top_k, int64_t num_experts,
                                 int64_t tile_expert_count, int has_sort_keys, int64_t n_sort_keys);

/* PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:97-117): token-major pair records
 * from the router's idx [tokens, top_k] u32 and w [tokens, top_k] FP16. */
int nvmai_hip_prefill_make_pairs(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint32_t* idx,
                                 const uint16_t* w, uint32_t tokens, uint32_t top_k,
                                 nvmai_prefill_pair* pairs);

/* PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:91-192) on the device:
 * pairs in any order -> pairs sorted by (sort key of the expert, expert, token, rank), the
 * per-expert offsets and counts, the groups and the tiles of <= tile_expert_count groups.
 * sort_keys: optional device u64 [num_experts].  A failing nvmai_prefill_grouping_check
 * returns NVMAI_ERR_INVALID_ARG; per-pair failures are found on the device and land in
 * info[2..3] (the arrays are then unspecified but every index in them is in range). */
int nvmai_hip_prefill_group_pairs(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_prefill_pair* pairs,
                                  uint64_t n_pairs, uint32_t query_count, uint32_t top_k,
                                  uint32_t num_experts, uint32_t tile_expert_count,
                                  const uint64_t* sort_keys, uint64_t n_sort_keys,
                                  const nvmai_prefill_grouping* out);

/* makeTokenExpertPairs + groupTokenExpertPairs in one step, straight from the router's
 * idx / w (RealPrefillRunner's use of the two, without the host round trip between). */
int nvmai_hip_prefill_group_routes(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint32_t* idx,
                                   const uint16_t* w, uint32_t query_count, uint32_t top_k,
                                   uint32_t num_experts, uint32_t tile_expert_count,
                                   const uint64_t* sort_keys, uint64_t n_sort_keys,
                                   const nvmai_prefill_grouping* out);

/* PrefillGroupedRoutedMoE.encodeStreamedBatched over every tile
 * (PrefillGroupedRoutedMoE.swift:413-489; kernels prefill.metal:460-534) with all experts
 * resident: act[p, :] = silu(gate_e x_token(p)) * (up_e x_token(p)) for sorted pair p, then
 * route_partials[token*top_k + rank, :] = down_e act[p, :], both rounded to the activation
 * type.  hidden [query_count, hidden_stride]; act_scratch [n_pairs, f] and route_partials
 * [n_pairs, d] are caller-owned, 16-bit.  d and f must be multiples of 64.  The kernel addresses
 * each operand array with 32-bit byte offsets: hidden, act_scratch, an expert's blob and one weight
 * matrix must each span less than 4 GiB (NVMAI_ERR_UNSUPPORTED otherwise).
 * A grouping whose validation failed on the device (grouping->info[2] != 0, where the reference
 * throws before any compute) runs no product: the call still returns NVMAI_OK, because the
 * failure is only known on the device, and route_partials is filled with zeros.  Read info[2]
 * after synchronising before trusting the outputs. */
int nvmai_hip_prefill_grouped_moe(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* experts_base,
                                  uint64_t expert_stride, const nvmai_expert_offsets* off, uint32_t bits,
                                  uint32_t d, uint32_t f, uint32_t num_experts, const void* hidden,
                                  uint32_t hidden_stride, uint32_t query_count, uint32_t top_k,
                                  const nvmai_prefill_grouping* grouping, void* act_scratch,
                                  void* route_partials);

/* PrefillGroupedRoutedMoEStreamedParams (PrefillGroupedRoutedMoE.swift:104-183 == prefill.metal:231-264):
 * the per-tile parameter block, 128 bytes, field for field (the reference's layout test:
 * PrefillGroupedRoutedMoETests+Layout.swift:7-30).  local_expert[i] = global id of the expert in
 * local slot i, 0xFFFFFFFF for the unused slots. */
typedef struct {
    uint32_t pair_start, pair_count, d, routed_intermediate, top_k, hidden_stride_elements, live_expert_count;
    uint32_t local_expert[16];
    uint32_t gate_w_off, gate_s_off, gate_b_off, up_w_off, up_s_off, up_b_off, down_w_off, down_s_off, down_b_off;
} nvmai_prefill_streamed_params;

/* PrefillGroupedRoutedMoE.encodeStreamedBatched for ONE tile (PrefillGroupedRoutedMoE.swift:413-489) with
 * the tile's experts bound one by one, as PrefillStreamedTileBinding (:185-323) binds the buffers
 * they were fetched into: expert_blobs is a HOST array of params->live_expert_count device pointers,
 * blob i = the expert params->local_expert[i] (16-byte aligned, any offset inside a larger buffer).
 * Runs gate/up + SwiGLU and down over the sorted pairs [pair_start, pair_start + pair_count) and
 * writes act_scratch[p, :] and route_partials[token * top_k + rank, :] for exactly those pairs;
 * sorted_pairs is the whole sorted array (n_sorted_pairs records), hidden [tokens,
 * hidden_stride_elements].  The binding's own checks (1..16 experts, unique ids) and the pair
 * range return NVMAI_ERR_INVALID_ARG; a pair whose expert is not bound (validateCoversPairs,
 * :274-287) is found on the device: nothing is computed and err (optional, 2 device words) =
 * (1, index of the first such pair), else (0, 0).  Same kernels as nvmai_hip_prefill_grouped_moe. */
int nvmai_hip_prefill_grouped_moe_streamed(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                           const nvmai_prefill_streamed_params* params,
                                           const void* const* expert_blobs, uint32_t bits, const void* hidden,
                                           const nvmai_prefill_pair* sorted_pairs, uint64_t n_sorted_pairs,
                                           void* act_scratch, void* route_partials, uint32_t* err);

/* MPPPrefillInt4QMM.encode (MPPPrefillInt4QMM.swift:63-128; kernel tensorops.metal:29-121):
 * the dense prefill product y[m, n] = x[m, k] . W[n, k]^T for m rows of activations against
 * one affine 4/8-bit matrix (group 64 along k, BF16 scale/bias), on the matrix cores: weights
 * dequantized once into MFMA operands, fp32 accumulate, y rounded to the activation type.
 * k must be a multiple of 64; x, y and the code rows 16-byte aligned; x and the code matrix each
 * below 4 GiB (NVMAI_ERR_UNSUPPORTED otherwise). */
int nvmai_hip_affine_qmm(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                         const uint16_t* scales, const uint16_t* biases, uint32_t bits, const void* x,
                         uint32_t x_stride, void* y, uint32_t y_stride, uint32_t m, uint32_t n, uint32_t k);

/* PrefillMoE.encodeReduceTokenMajor (PrefillMoE.swift:11-40; prefill.metal:437-458):
 * h2[t, :] = sum over ranks, in rank order, of fma(w[t, r], route_partials[t*top_k + r, :]). */
int nvmai_hip_prefill_moe_reduce_token_major(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                             const void* route_partials, const uint16_t* route_weights,
                                             void* h2, uint32_t h2_stride, uint32_t query_count,
                                             uint32_t top_k, uint32_t d);


/* ---- KV cache -------------------------------------------------------------------------- */

/* KVCacheManager.rowLayout (KVCacheManager.swift:437-446): bytes per token row and bytes of
 * packed codes for `elements` = num_kv_heads * head_dim values at `bits` in {4, 8, 16}.
 * Row = codes | FP16 scales[groups] | FP16 biases[groups], groups of 64.  Host arithmetic. */
int nvmai_kv_row_layout(uint32_t elements, uint32_t bits, uint32_t* stride, uint32_t* value_bytes);

/* KVView (KVCacheManager.swift:19-31) without the Metal buffer: where a layer's K or V rows
 * live and how they are encoded. */
typedef struct {
    void* base;            /* row of position p at base + p * stride */
    uint32_t stride;
    uint32_t value_bytes;
    uint32_t bits;         /* KVCachePrecision raw value: 4, 8 or 16 (RuntimeConfiguration.swift:81-88) */
    uint32_t group_size;   /* 64 */
} nvmai_kv_view;

/* KVCacheQuantizer.encode (KVCacheQuantizer.swift:13-50; kernel kv_cache_quantize.metal:7-73):
 * quantize token_count rows of element_count activations (row t at source + t *
 * source_stride elements) into destination rows 0..token_count-1. */
int nvmai_hip_kv_quantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* source,
                                 uint32_t source_stride, const nvmai_kv_view* destination,
                                 uint32_t token_count, uint32_t element_count);

/* RoPE.encodeNeoxSubdim (RoPE.swift:48; kernel rope.metal:80-102), in place on
 * data[tokens, heads, head_dim].  positions: optional device array of one position per token;
 * NULL = every token at `position` (the reference's single-position call). */
int nvmai_hip_rope_neox_subdim(nvmai_hip_ctx* ctx, nvmai_stream stream, void* data, uint32_t tokens,
                               uint32_t heads, uint32_t head_dim, uint32_t rotary_dim,
                               const uint32_t* positions, uint32_t position, float theta);

/* Attention.encodeFull / encodeSWA (Attention.swift:207-239, 170-205; kernels
 * attention.metal:163-261, 388-429) with a batch dimension: one query token per sequence,
 * q and out are [batch, num_q_heads, head_dim] activations, sequence b reads rows
 * [kv_start, seq_len) of k->base + b * kv_batch_stride (same for v).  scale <= 0 selects
 * 1/sqrt(head_dim) (Attention.defaultScale).  seq_len == kv_start writes zeros. */
int nvmai_hip_attention_decode(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                               const nvmai_kv_view* k, const nvmai_kv_view* v,
                               uint64_t kv_batch_stride, void* out, uint32_t batch,
                               uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                               uint32_t seq_len, uint32_t kv_start, float scale);

/* nvmai_hip_attention_decode followed by Elementwise.encodeSigmoidGateMul over its output
 * (RealForwardRunner.swift:2257-2276; utility.metal:47-58) in the same launches:
 * out = round(attention) / (1 + exp(-gate)), gate rows [batch, gate_stride] activations laid out
 * like out.  Same bits as the two calls one after the other. */
int nvmai_hip_attention_decode_gated(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                     const nvmai_kv_view* k, const nvmai_kv_view* v,
                                     uint64_t kv_batch_stride, void* out, const void* gate,
                                     uint32_t gate_stride, uint32_t batch, uint32_t head_dim,
                                     uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                                     uint32_t kv_start, float scale);

/* The same call for sequences of different lengths: sequence b reads rows
 * [kv_starts[b], min(seq_lens[b], max_seq_len)) of its cache (kv_starts NULL: from row 0).
 * seq_lens and kv_starts are device arrays of `batch` words read by the kernels, so a captured
 * graph follows them; max_seq_len bounds every row the call may touch and sizes the chunking.
 * The reference issues one encodeFull per sequence (Attention.swift:207-239); an empty range
 * writes zeros as there. */
int nvmai_hip_attention_decode_ragged(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                      const nvmai_kv_view* k, const nvmai_kv_view* v,
                                      uint64_t kv_batch_stride, void* out, uint32_t batch,
                                      uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                      const uint32_t* seq_lens, const uint32_t* kv_starts,
                                      uint32_t max_seq_len, float scale);

/* PrefillAttention.encodeCausal on the causalTiled path (PrefillAttention.swift:97-167; kernel
 * attention_prefill_causal_tiled, prefill.metal:709-830) over fp16, 8-bit or 4-bit K/V rows:
 * query token t of the chunk (row q + t * q_token_stride elements, [num_q_heads, head_dim]) sits
 * at absolute position start_position + t and attends to the keys
 * [first, min(kv_valid_count, start_position + t + 1)), first = max(0, start_position + t + 1 -
 * sliding_window) when sliding_window != 0, else 0; its output row is out + t * o_token_stride
 * elements.  kv_ring_capacity != 0: the row of key p is p % kv_ring_capacity (function constant
 * 76 of the reference).  Errors follow PrefillAttention.validate (PrefillAttention.swift:169-191):
 * strides below num_q_heads * head_dim, query_count == 0, or start_position + query_count >
 * kv_valid_count give NVMAI_ERR_INVALID_ARG.  scale <= 0 selects 1/sqrt(head_dim).
 * A chunk with head_dim 256, a power-of-two group size and enough queries to give every compute
 * unit a block (query_count * num_q_heads >= 16,384), its q and out rows at 16-byte boundaries,
 * runs in two launches: the key range is dequantized once into fp16 scratch in the context's
 * workspace (1,024 bytes per key and kv head), then a flash-attention kernel works on that.  Size
 * the workspace with an eager call or nvmai_hip_ctx_reserve before capturing such a call into a
 * graph (a captured call that would have to grow it returns NVMAI_ERR_SCRATCH). */
int nvmai_hip_attention_prefill_causal(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                       uint32_t q_token_stride, const nvmai_kv_view* k,
                                       const nvmai_kv_view* v, void* out, uint32_t o_token_stride,
                                       uint32_t start_position, uint32_t query_count,
                                       uint32_t kv_valid_count, uint32_t sliding_window,
                                       uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                       uint32_t kv_ring_capacity, float scale);

/* Attention.splitGeometry (Attention.swift:148-168): the reference's chunking of a KV range,
 * reported for callers that size scratch the way it does.  Host arithmetic. */
int nvmai_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                                   uint32_t kv_start, int prefer_gqa_swa, uint32_t* effective_length,
                                   uint32_t* num_chunks, uint32_t* chunk_length,
                                   uint32_t* partial_threadgroups);

/* ---- logits -> token --------------------------------------------------------------------- */

/* LogitSoftcapSoftmaxTiled.encode (LogitOutput.swift:90-141; kernels logit.metal:155-257):
 * probs[r, :] = softmax(softcap(logits[r, :])) as FP16 for `rows` rows of v activations.
 * softcap <= 0 disables the cap. */
int nvmai_hip_softmax_tiled(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* logits,
                            uint32_t logits_stride, uint16_t* probs, uint32_t probs_stride,
                            uint32_t rows, uint32_t v, float softcap);

/* SampleTopK64.encode (LogitOutput.swift:267-333; kernels logit.metal:628-758): one token per
 * row from the top `top_k` (1..64) of FP16 probs with top-p and temperature (> 0); seeds is a
 * HOST array of one xorshift64* seed per row (rows <= 32).  top64_out (optional, device):
 * per row the 64 sorted candidates as (float bits, index) u32 pairs. */
int nvmai_hip_sample_topk64(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint16_t* probs,
                            uint32_t probs_stride, uint32_t rows, uint32_t v, float temperature,
                            float top_p, const uint64_t* seeds, uint32_t top_k, uint32_t* out_token,
                            uint32_t* top64_out);

/* Sample.encode (LogitOutput.swift:157-199; kernel logit.metal:315-585), the kernel's three
 * paths: temperature <= 0 is greedy argmax (lowest index wins ties); top_k == 0 with top_p
 * outside (0, 1) is the Gumbel-max draw argmax(log p / T + g) with g from SplitMix64 of
 * (seed, position, index) (logit.metal:296-313, 391-429); otherwise top_k (0 = none, capped at
 * 256) argmax passes and the top-p / temperature / inverse-CDF draw with xorshift64*.
 * seeds: HOST array, one per row; positions: HOST array, one per row, NULL = 0 (only the
 * Gumbel path reads it); rows <= 32. */
int nvmai_hip_sample(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint16_t* probs,
                     uint32_t probs_stride, uint32_t rows, uint32_t v, float temperature,
                     uint32_t top_k, float top_p, const uint64_t* seeds, const uint32_t* positions,
                     uint32_t* out_token);

/* Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293) on the device, in place on one row
 * of `v` logits (activations): for every distinct id of history_ids (device int32 [n_ids]; ids
 * outside the vocabulary are skipped, repeats count once) a positive logit is divided by
 * `penalty`, a negative one multiplied; with logit_softcap > 0 the penalty acts on the capped
 * logit and is mapped back through atanh.  penalty == 1 or n_ids == 0 does nothing. */
int nvmai_hip_repetition_penalty(nvmai_hip_ctx* ctx, nvmai_stream stream, void* logits, uint32_t v,
                                 const int32_t* history_ids, uint32_t n_ids, float penalty,
                                 float logit_softcap);

/* GenerationConfig (Sampler.swift:19-81), the fields Sampler.sample reads.  top_k 0 and top_p 0
 * stand for the reference's nil (no top-k cap; top-p 1.0); has_seed 0 = clock-derived seed. */
typedef struct {
    float temperature;          /* >= 0; 0 = greedy */
    int32_t top_k;              /* 0 = nil, else 1..256 */
    float top_p;                /* 0 = nil, else (0, 1] */
    float repetition_penalty;   /* 1 = off */
    uint64_t seed;
    int32_t has_seed;
} nvmai_generation_config;
enum { NVMAI_SAMPLER_TILED = 0, NVMAI_SAMPLER_GENERIC = 1 };                     /* RuntimeSamplerPath */
enum { NVMAI_SAMPLE_PATH_GREEDY = 0, NVMAI_SAMPLE_PATH_SAMPLED = 1, NVMAI_SAMPLE_PATH_PENALTY = 2 };   /* SamplePath */

/* Sampler.sample (Sampler.swift:171-234) for one row: the repetition penalty over the history
 * (when the penalty is not 1 and the history is not empty; edits `logits` in place), softcap +
 * softmax into probs (FP16 [v] scratch), then the tiled top-64 sampler when sampler_path is
 * NVMAI_SAMPLER_TILED, temperature > 0, top_k is 1..64 and v is within that sampler's 262,144,
 * else the generic kernel (greedy at
 * temperature 0, Gumbel-max without top-k and top-p, k argmax passes otherwise), with the seed
 * of Sampler.seedFor(config, position).  path_taken (optional, host) receives the SamplePath.
 * A configuration GenerationConfig.validate refuses returns NVMAI_ERR_INVALID_ARG; top_p below
 * one without top_k returns NVMAI_ERR_UNSUPPORTED, as it throws there. */
int nvmai_hip_sampler_sample(nvmai_hip_ctx* ctx, nvmai_stream stream, void* logits, uint16_t* probs,
                             uint32_t v, const int32_t* history_ids, uint32_t n_history,
                             const nvmai_generation_config* config, int64_t position,
                             float logit_softcap, int sampler_path, uint32_t* out_token,
                             int* path_taken);

/* ---- the small operators around the MoE block of a decode step ---------------------------- */

/* RMSNorm.encodeBF16W / encodeNoScale / encodeBF16WPerHead / encodeNoScalePerHead
 * (RMSNorm.swift:52-142; kernels rmsnorm.metal:64-175): out[r] = x[r] * inv_r * weight with
 * inv_r = 1 / sqrt(mean(x[r]^2) + eps), fp32 arithmetic, 16-bit activations in and out; row r
 * at x + r * x_stride elements (the per-head kernels: rows = heads, strides = head_dim).
 * weight: BF16 [d] shared by all rows, NULL = no scale.  out may be x (in place). */
int nvmai_hip_rmsnorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* x, uint32_t x_stride,
                      const uint16_t* weight, void* out, uint32_t out_stride, uint32_t rows,
                      uint32_t d, float eps);

/* Elementwise (Elementwise.swift:28-121; kernels utility.metal:32-121) and the SwiGLU product of the
 * shared expert (SharedExpertInt4.swift:61-96, silu_mul_fp16): 16-bit activations, fp32 arithmetic.
 *   silu_mul:           out[i] = silu(gate[i]) * up[i]
 *   sigmoid_gate_mul:   out[i] = out[i] * sigmoid(gate[i])          (in place)
 *   sigmoid_scalar_mul: y[i]   = y[i] * sigmoid(gate[0])            (in place)
 *   residual_add:       hidden[i] = hidden[i] + delta[i]            (in place)
 *   split_q_gate:       packed [heads, 2 dim] -> q [heads, dim], gate [heads, dim]
 *   concat_rows:        lhs, rhs [rows, dim] -> out [rows, 2 dim] */
int nvmai_hip_silu_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* gate, const void* up,
                       void* out, uint32_t count);
int nvmai_hip_sigmoid_gate_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, void* out, const void* gate,
                               uint32_t count);
int nvmai_hip_sigmoid_scalar_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, void* y, const void* gate,
                                 uint32_t count);
int nvmai_hip_residual_add(nvmai_hip_ctx* ctx, nvmai_stream stream, void* hidden, const void* delta,
                           uint32_t count);
int nvmai_hip_split_q_gate(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* packed, void* q,
                           void* gate, uint32_t heads, uint32_t dim);
int nvmai_hip_concat_rows(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* lhs, const void* rhs,
                          void* out, uint32_t rows, uint32_t dim);

/* AffineQuantEmbeddingLookup.encode (kernel embed_lookup_int4, dequant_int4.metal:63-91; a block
 * of tokens: prefill_embed_lookup_affine_block, prefill.metal:59): out[t] = (q * scale + bias) *
 * out_scale for row token[t] of a 4- or 8-bit affine table [vocab, d]; a token id >= vocab gives
 * a row of zeros.  token_ids: device array of n_tokens ids, or NULL = the single id `token_id`
 * for every row (the reference passes the id by value). */
int nvmai_hip_embed_lookup(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* table,
                           const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                           const uint32_t* token_ids, uint32_t token_id, uint32_t n_tokens, void* out,
                           uint32_t out_stride, uint32_t d, uint32_t vocab, float out_scale);

/* LMHeadChainInt4.encodeGreedyDecode (LMHeadChainInt4.swift:58-130; kernels rmsnorm_bf16w,
 * lm_head_greedy_int4_rows_chunk_raw, lm_head_greedy_int4_rows_reduce, logit.metal:761-937):
 * out_tokens[t] = argmax over the rows of a 4- or 8-bit affine LM head [vocab, d] of
 * W[row] . RMSNorm(hidden[t]), over the finite logits only, ties to the lower index, 0 when no
 * logit is finite.  norm_weight: BF16 [d], NULL = hidden is used as it is.  Rows of at most
 * 2048 bytes (d <= 2048 at 8 bit, 4096 at 4 bit). */
int nvmai_hip_lm_head_greedy(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* hidden,
                             uint32_t hidden_stride, uint32_t n_tokens, const uint16_t* norm_weight,
                             const uint8_t* weights, const uint16_t* scales, const uint16_t* biases,
                             uint32_t bits, uint32_t* out_tokens, uint32_t d, uint32_t vocab,
                             float rms_eps);

/* hidden[r] += delta[r] (Elementwise.encodeResidualAdd, utility.metal:95-104), then
 * out[r] = RMSNorm(hidden[r]) * weight (RMSNorm.encodeBF16W, rmsnorm.metal:64-110): the residual add
 * that ends one block of a layer and the norm that opens the next (RealForwardRunner.swift:1897-1905)
 * in one launch, same results as the two calls.  weight: BF16 [d] or NULL. */
int nvmai_hip_residual_add_rmsnorm(nvmai_hip_ctx* ctx, nvmai_stream stream, void* hidden, uint32_t hidden_stride,
                                   const void* delta, uint32_t delta_stride, const uint16_t* weight, void* out,
                                   uint32_t out_stride, uint32_t rows, uint32_t d, float eps);

/* nvmai_hip_residual_add_rmsnorm followed by nvmai_hip_affine_gemv over the normed rows -- the input
 * norm of a layer and its fused input projection (RealForwardRunner.swift:1857-1875, 2066-2085) -- in ONE
 * launch for up to four rows of at most 2048 elements against a projection of at most 16,384 rows:
 * every block norms the rows for itself (same arithmetic and order, so the same bits), the first
 * block stores the updated residual rows to hidden_out, which must not be `hidden` (other blocks
 * still read it).  delta may be NULL (norm only).  Any other shape runs the steps one after the other
 * through normed_scratch ([n_tokens, normed_stride] activations; NVMAI_ERR_UNSUPPORTED when NULL). */
int nvmai_hip_affine_gemv_prenorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                                  const uint16_t* scales, const uint16_t* biases, uint32_t bits, const void* hidden,
                                  uint32_t hidden_stride, const void* delta, uint32_t delta_stride,
                                  const uint16_t* norm_weight, float eps, void* hidden_out,
                                  uint32_t hidden_out_stride, void* normed_scratch, uint32_t normed_stride,
                                  uint32_t n_tokens, uint32_t m, uint32_t n, void* y, uint32_t y_stride);

/* The epilogue of the q / k / v projection of a full-attention layer in one launch:
 * Elementwise.encodeSplitQGate + RMSNorm.encodeBF16WPerHead (q, k) + RoPE.encodeNeoxSubdim (q, k)
 * (RealForwardRunner.swift:2213-2255), or with q_packed = 0 and v_norm = 1 the reference's own
 * FusedQKVEpilogue (fused.metal:72-162).  proj: [tokens, proj_stride] activations, per token the q
 * heads (packed [q ; gate] pairs of 2 head_dim when q_packed), then the k heads, then the v heads, as the
 * fused projection writes them.  q_out, gate_out: [tokens, num_q_heads, head_dim]; k_out, v_out:
 * [tokens, kv_stride] stage rows for nvmai_hip_kv_quantize_affine.  positions: device array of one
 * position per token, or NULL = `position` for all.  Same bits as the separate calls.  head_dim <= 512. */
int nvmai_hip_attn_qkv_epilogue(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* proj, uint32_t proj_stride,
                                int q_packed, const uint16_t* q_weight, const uint16_t* k_weight, void* q_out,
                                void* gate_out, void* k_out, void* v_out, uint32_t kv_stride, uint32_t tokens,
                                uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, uint32_t rotary_dim,
                                int v_norm, const uint32_t* positions, uint32_t position, float theta, float eps);

/* The same epilogue with KVCacheQuantizer.encode (KVCacheQuantizer.swift:17-60;
 * kv_cache_quantize.metal:7-73) of the finished k and v rows in the same launch: token t's rows
 * go to k_cache->base + t * k_cache->stride and v_cache->base + t * v_cache->stride as
 * [codes | fp16 scales | fp16 biases] (4 or 8 bit, group 64; head_dim a multiple of 64; both views of
 * one format).  k_out / v_out (the 16-bit stage rows) may both be NULL.  Same bits as
 * nvmai_hip_attn_qkv_epilogue followed by two nvmai_hip_kv_quantize_affine calls. */
int nvmai_hip_attn_qkv_epilogue_kv(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* proj, uint32_t proj_stride,
                                   int q_packed, const uint16_t* q_weight, const uint16_t* k_weight, void* q_out,
                                   void* gate_out, void* k_out, void* v_out, uint32_t kv_stride,
                                   const nvmai_kv_view* k_cache, const nvmai_kv_view* v_cache, uint32_t tokens,
                                   uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, uint32_t rotary_dim,
                                   int v_norm, const uint32_t* positions, uint32_t position, float theta, float eps);

/* ---- gated-DeltaNet linear attention ------------------------------------------------------- */

/* LinearAttentionConfig (ModelTypes.swift:15-41).  Rows of qkv / conv_out are
 * [q: Hk * Dk][k: Hk * Dk][v: Hv * Dv]. */
typedef struct {
    uint32_t num_k_heads, num_v_heads, key_head_dim, value_head_dim, conv_kernel_size;
} nvmai_gdn_config;

/* GDN.encodeConvDecode / encodeConvPrefill + encodeConvTailUpdate + encodeQKNorm (GDN.swift:130-246;
 * kernels gdn.metal:241-366, 386-441): conv_out = silu(causal depthwise conv of [tail | rows]),
 * then the q and k heads normalised without weight and scaled by 1 / Dk and 1 / sqrt(Dk), and the
 * tail replaced by the last K - 1 raw rows.  `batch` sequences of `rows` tokens each (1 = a decode
 * step): qkv_raw and conv_out are [batch * rows, stride] activations, tail is [batch, K - 1, C]
 * activations, conv_weight BF16 [C, K].  K <= 8. */
int nvmai_hip_gdn_conv_norm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                            const void* qkv_raw, uint32_t qkv_stride, void* tail, const uint16_t* conv_weight,
                            void* conv_out, uint32_t conv_out_stride, uint32_t rows, uint32_t batch);

/* GDN.encodeDeltaStepDecode / encodeDeltaStepPrefill + encodeGatedNorm (GDN.swift:248-341; kernels
 * gdn.metal:443-587, 589-642): the gated delta rule over the rows of each sequence in order, state
 * [batch, Hv, Dv, Dk] updated in place -- fp32 as the reference keeps it, or BF16 when
 * state_is_bf16 (half the bytes per token, arithmetic still fp32) -- and
 * out = rmsnorm(y) * norm_weight * silu(z) per value head.  a_proj, b_proj: [batch * rows, ab_stride]
 * activations; a_log, dt_bias: BF16 [Hv]; z, out: [batch * rows, stride] activations; norm_weight
 * BF16 [Dv].  (Dk, Dv) in {(128, 128), (64, 64), (32, 32), (64, 128), (128, 64)}.
 * A call of 64 rows or more over 128 x 128 heads takes sixteen rows at a time on the matrix cores and needs
 * workspace: 2,304 bytes per (sequence, value head, sixteen rows), and in a BF16 context 8,192 bytes more per
 * (sequence, value head, sixteen rows) plus 4,096 per (sequence, key head, sixteen rows) -- 103 MB for one
 * sequence of 4096 rows with 32 value and 16 key heads.  Under stream capture that workspace must
 * already be there (nvmai_hip_ctx_reserve, or the same call made eagerly once), else the call returns
 * NVMAI_ERR_SCRATCH and launches nothing -- it does not fall back to the row-by-row kernels, whose summation
 * order (and so the last bits) would differ from the eager call's. */
int nvmai_hip_gdn_delta_gated_norm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                                   const void* conv_out, uint32_t conv_out_stride, const void* a_proj,
                                   const void* b_proj, uint32_t ab_stride, const uint16_t* a_log,
                                   const uint16_t* dt_bias, void* state, int state_is_bf16, const void* z,
                                   uint32_t z_stride, const uint16_t* norm_weight, void* out, uint32_t out_stride,
                                   uint32_t rows, uint32_t batch);

/* One decode token per sequence: nvmai_hip_gdn_conv_norm followed by nvmai_hip_gdn_delta_gated_norm
 * (rows = 1) in ONE launch -- a block per (key head, sequence) runs the conv of its q / k channels
 * once and the delta rule of each of its Hv / Hk value heads, and shifts its tail columns in place.
 * Same bits as the two calls (out, state, tail).  Fused for (Dk, Dv) in {(128, 128), (32, 32)} with
 * Hv / Hk in {1, 2}; any other shape runs the two kernels through conv_scratch ([batch,
 * conv_scratch_stride] activations), and returns NVMAI_ERR_UNSUPPORTED when that is NULL. */
int nvmai_hip_gdn_decode_step(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                              const void* qkv_raw, uint32_t qkv_stride, void* tail, const uint16_t* conv_weight,
                              void* conv_scratch, uint32_t conv_scratch_stride, const void* a_proj,
                              const void* b_proj, uint32_t ab_stride, const uint16_t* a_log, const uint16_t* dt_bias,
                              void* state, int state_is_bf16, const void* z, uint32_t z_stride,
                              const uint16_t* norm_weight, void* out, uint32_t out_stride, uint32_t batch);

/* GDN.encodeInputProjections (GDN.swift:85-128; kernel gdn_in_proj_gemv_simd, gdn.metal:179-239) and
 * FusedQKVGEMV.encode (kernel dequant_int4_qkv_gemv_simd, dequant_int4.metal:279-329): several
 * projections of the same input rows.  parts[i]: y_i = W_i x.  When the parts' codes, scales,
 * biases and outputs each lie back to back in memory (and there is one input row) the call is ONE
 * launch over the concatenated rows; otherwise one launch per part.  Same results either way. */
typedef struct {
    const uint8_t* weights;
    const uint16_t* scales;
    const uint16_t* biases;
    uint32_t rows;
    void* y;                /* activations [n_tokens, y_stride] */
    uint32_t y_stride;
} nvmai_gemv_part;
int nvmai_hip_affine_gemv_fused(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gemv_part* parts,
                                uint32_t n_parts, uint32_t bits, const void* x, uint32_t x_stride,
                                uint32_t n_tokens, uint32_t n);

/* Sampler.seedFor (Sampler.swift:304-325): splitmix64(seed + position), 0 mapped away. */
uint64_t nvmai_sampler_seed_for(uint64_t seed, int64_t position);

#ifdef __cplusplus
}
#endif
#endif /* NVMAI_HIP_H */
