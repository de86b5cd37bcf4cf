// Entry points: RMSNorm, the elementwise helpers of the layer loop, affine embedding lookup, fused greedy LM head.
#include <initializer_list>

#include "ctx.hpp"
#include "step_kernels.hpp"

using namespace nvmai;

namespace {
// Rows travel through LDS when they can be moved 16 bytes at a time: four rows and the weight, 10 d bytes.
bool rms_staged_ok(const void* a, uint32_t a_stride, const void* b, uint32_t b_stride, const void* c, uint32_t c_stride,
                   const void* weight, uint32_t d) {
    return d % 8 == 0 && d <= 6144 && aligned16(a) && a_stride % 8 == 0 && (!b || (aligned16(b) && b_stride % 8 == 0)) &&
           aligned16(c) && c_stride % 8 == 0 && (!weight || aligned16(weight));
}
// Up to this many 2048-wide rows take one wave per block and row with no LDS (rms_direct_kernel).
constexpr uint32_t RMS_DIRECT_ROWS = 256;
}  // namespace

extern "C" int nvmai_hip_rmsnorm(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* x, uint32_t x_stride,
                                 const uint16_t* weight, void* out, uint32_t out_stride, uint32_t rows,
                                 uint32_t d, float eps) {
    if (!ctx || !x || !out || d == 0 || x_stride < d || out_stride < d) return NVMAI_ERR_INVALID_ARG;
    if (rows == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((rows + 3) / 4);
    const bool staged = rms_staged_ok(x, x_stride, nullptr, 0, out, out_stride, weight, d);
    const size_t lds = staged ? (size_t)d * 10 : 0;
    const bool direct = d == 2048 && rows <= RMS_DIRECT_ROWS;
#define NVMAI_RMS(ACT)                                                                                              \
    do {                                                                                                            \
        if (direct) rms_direct_kernel<ACT, 2048, false><<<rows, 64, 0, s>>>((uint16_t*)x, x_stride, nullptr, 0, weight, (uint16_t*)out, out_stride, eps); \
        else if (staged && d == 2048) rmsnorm_kernel<ACT, true, 2048><<<grid, 256, lds, s>>>((const uint16_t*)x, x_stride, weight, (uint16_t*)out, out_stride, rows, d, eps); \
        else if (staged) rmsnorm_kernel<ACT, true, 0><<<grid, 256, lds, s>>>((const uint16_t*)x, x_stride, weight, (uint16_t*)out, out_stride, rows, d, eps); \
        else rmsnorm_kernel<ACT, false, 0><<<grid, 256, 0, s>>>((const uint16_t*)x, x_stride, weight, (uint16_t*)out, out_stride, rows, d, eps);        \
    } while (0)
    if (ctx->act == ACT_BF16) NVMAI_RMS(ACT_BF16); else NVMAI_RMS(ACT_FP16);
#undef NVMAI_RMS
    return launch_status();
}

extern "C" int nvmai_hip_residual_add_rmsnorm(nvmai_hip_ctx* ctx, nvmai_stream stream, void* hidden,
                                              uint32_t hidden_stride, const void* delta, uint32_t delta_stride,
                                              const uint16_t* weight, void* out, uint32_t out_stride, uint32_t rows,
                                              uint32_t d, float eps) {
    if (!ctx || !hidden || !delta || !out || d == 0 || hidden_stride < d || delta_stride < d || out_stride < d)
        return NVMAI_ERR_INVALID_ARG;
    if (rows == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((rows + 3) / 4);
    const bool staged = rms_staged_ok(hidden, hidden_stride, delta, delta_stride, out, out_stride, weight, d);
    const size_t lds = staged ? (size_t)d * 10 : 0;
    const bool direct = d == 2048 && rows <= RMS_DIRECT_ROWS;
#define NVMAI_RES(ACT)                                                                                              \
    do {                                                                                                            \
        if (direct) rms_direct_kernel<ACT, 2048, true><<<rows, 64, 0, s>>>((uint16_t*)hidden, hidden_stride, (const uint16_t*)delta, delta_stride, weight, (uint16_t*)out, out_stride, eps); \
        else if (staged && d == 2048) residual_add_rmsnorm_kernel<ACT, true, 2048><<<grid, 256, lds, s>>>((uint16_t*)hidden, hidden_stride, (const uint16_t*)delta, delta_stride, weight, (uint16_t*)out, out_stride, rows, d, eps); \
        else if (staged) residual_add_rmsnorm_kernel<ACT, true, 0><<<grid, 256, lds, s>>>((uint16_t*)hidden, hidden_stride, (const uint16_t*)delta, delta_stride, weight, (uint16_t*)out, out_stride, rows, d, eps); \
        else residual_add_rmsnorm_kernel<ACT, false, 0><<<grid, 256, 0, s>>>((uint16_t*)hidden, hidden_stride, (const uint16_t*)delta, delta_stride, weight, (uint16_t*)out, out_stride, rows, d, eps);        \
    } while (0)
    if (ctx->act == ACT_BF16) NVMAI_RES(ACT_BF16); else NVMAI_RES(ACT_FP16);
#undef NVMAI_RES
    return launch_status();
}

namespace {
int qkv_epilogue_impl(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* proj, uint32_t proj_stride, int q_packed,
                      const uint16_t* q_weight, const uint16_t* k_weight, void* q_out, void* gate_out, void* k_out,
                      void* v_out, uint32_t kv_stride, uint32_t tokens, uint32_t num_q_heads, uint32_t num_kv_heads,
                      uint32_t head_dim, uint32_t rotary_dim, int v_norm, const uint32_t* positions, uint32_t position,
                      float theta, float eps, const nvmai_kv_view* k_cache, const nvmai_kv_view* v_cache) {
    const bool cached = k_cache || v_cache;
    if (!ctx || !proj || !q_out || (q_packed && !gate_out)) return NVMAI_ERR_INVALID_ARG;
    if (cached ? (!k_cache || !v_cache) : (!k_out || !v_out)) return NVMAI_ERR_INVALID_ARG;
    if ((k_out == nullptr) != (v_out == nullptr)) return NVMAI_ERR_INVALID_ARG;
    if (head_dim == 0 || head_dim > 512 || num_q_heads == 0 || num_kv_heads == 0) return NVMAI_ERR_INVALID_ARG;   // kFusedMaxHeadDim
    if (rotary_dim > head_dim || (rotary_dim & 1u)) return NVMAI_ERR_INVALID_ARG;
    const uint32_t span = (q_packed ? 2u : 1u) * num_q_heads * head_dim + 2u * num_kv_heads * head_dim;
    if (proj_stride < span || (k_out && kv_stride < num_kv_heads * head_dim)) return NVMAI_ERR_INVALID_ARG;
    QkvEpilogueParams p{};
    if (cached) {
        // KVCacheQuantizer.encode's checks (KVCacheQuantizer.swift:17-30) on both destinations
        if (head_dim % 64) return NVMAI_ERR_UNSUPPORTED;      // a group must not straddle two heads
        uint32_t stride = 0, vb = 0;
        for (const nvmai_kv_view* c : {k_cache, v_cache}) {
            if (!c->base) return NVMAI_ERR_INVALID_ARG;
            if ((c->bits != 4 && c->bits != 8) || c->group_size != 64) return NVMAI_ERR_UNSUPPORTED;
            if (nvmai_kv_row_layout(num_kv_heads * head_dim, c->bits, &stride, &vb) != NVMAI_OK) return NVMAI_ERR_INVALID_ARG;
            if (c->value_bytes != vb || c->stride < stride || (c->stride & 1u)) return NVMAI_ERR_INVALID_ARG;
        }
        if (k_cache->bits != v_cache->bits || k_cache->stride != v_cache->stride) return NVMAI_ERR_INVALID_ARG;
        p.kc = (uint8_t*)k_cache->base; p.vc = (uint8_t*)v_cache->base;
        p.kv_bits = k_cache->bits; p.kv_row_stride = k_cache->stride; p.kv_value_bytes = k_cache->value_bytes;
    }
    if (tokens == 0) return NVMAI_OK;
    p.proj = (const uint16_t*)proj; p.proj_stride = proj_stride; p.q_packed = q_packed ? 1u : 0u;
    p.q_weight = q_weight; p.k_weight = k_weight;
    p.q_out = (uint16_t*)q_out; p.gate_out = (uint16_t*)gate_out; p.k_out = (uint16_t*)k_out; p.v_out = (uint16_t*)v_out;
    p.kv_stride = kv_stride; p.tokens = tokens; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim; p.rotary_dim = rotary_dim; p.v_norm = v_norm ? 1u : 0u;
    p.positions = positions; p.position0 = position; p.theta = theta; p.eps = eps;
    const dim3 grid((num_q_heads + 2 * num_kv_heads + 3) / 4, tokens);
    hipStream_t s = (hipStream_t)stream;
    if (head_dim == 256) {          // the production head: loops unrolled, a pass's loads in flight together
        if (ctx->act == ACT_BF16) qkv_epilogue_kernel<ACT_BF16, 256><<<grid, 256, 0, s>>>(p);
        else qkv_epilogue_kernel<ACT_FP16, 256><<<grid, 256, 0, s>>>(p);
    } else if (ctx->act == ACT_BF16) qkv_epilogue_kernel<ACT_BF16, 0><<<grid, 256, 0, s>>>(p);
    else qkv_epilogue_kernel<ACT_FP16, 0><<<grid, 256, 0, s>>>(p);
    return launch_status();
}
}  // namespace

extern "C" int nvmai_hip_attn_qkv_epilogue(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* proj,
                                           uint32_t proj_stride, int q_packed, const uint16_t* q_weight,
                                           const uint16_t* k_weight, void* q_out, void* gate_out, void* k_out,
                                           void* v_out, uint32_t kv_stride, uint32_t tokens, uint32_t num_q_heads,
                                           uint32_t num_kv_heads, uint32_t head_dim, uint32_t rotary_dim, int v_norm,
                                           const uint32_t* positions, uint32_t position, float theta, float eps) {
    return qkv_epilogue_impl(ctx, stream, proj, proj_stride, q_packed, q_weight, k_weight, q_out, gate_out, k_out, v_out,
                             kv_stride, tokens, num_q_heads, num_kv_heads, head_dim, rotary_dim, v_norm, positions,
                             position, theta, eps, nullptr, nullptr);
}

extern "C" int nvmai_hip_attn_qkv_epilogue_kv(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* proj,
                                              uint32_t proj_stride, int q_packed, const uint16_t* q_weight,
                                              const uint16_t* k_weight, void* q_out, void* gate_out, void* k_out,
                                              void* v_out, uint32_t kv_stride, const nvmai_kv_view* k_cache,
                                              const nvmai_kv_view* v_cache, uint32_t tokens, uint32_t num_q_heads,
                                              uint32_t num_kv_heads, uint32_t head_dim, uint32_t rotary_dim, int v_norm,
                                              const uint32_t* positions, uint32_t position, float theta, float eps) {
    if (!k_cache || !v_cache) return NVMAI_ERR_INVALID_ARG;
    return qkv_epilogue_impl(ctx, stream, proj, proj_stride, q_packed, q_weight, k_weight, q_out, gate_out, k_out, v_out,
                             kv_stride, tokens, num_q_heads, num_kv_heads, head_dim, rotary_dim, v_norm, positions,
                             position, theta, eps, k_cache, v_cache);
}

// Dense BF16 rows [m, n] against n_tokens BF16 inputs: the bits == 16 case of nvmai_hip_affine_gemv.
namespace nvmai {
int dense_bf16_gemv(nvmai_hip_ctx* ctx, hipStream_t s, const uint16_t* w, const void* x, uint32_t x_stride,
                    uint32_t n_tokens, uint32_t m, uint32_t n, void* y, float* y_f32, uint32_t y_stride) {
    if (ctx->act != ACT_BF16) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || n % 64 || n > 4096 || x_stride < n || y_stride < m) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(w) || !aligned16(x) || x_stride % 8) return NVMAI_ERR_ALIGNMENT;
    if (m == 0 || n_tokens == 0) return NVMAI_OK;
    static bool lds_raised = false;
    if (!lds_raised) {
        NVMAI_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(dense_bf16_gemv_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, DENSE_TOK * (4096 * 2 + 16)));
        lds_raised = true;
    }
    const uint32_t groups = (m + 63) / 64;                   // 64 rows per block pass
    // Blocks per compute unit follow from the staged inputs (4 KB of LDS each at the usual width):
    // five at one input, two at sixteen.  With three or more the hardware's own hand-out of short
    // blocks is the fastest form (one pass per block; two or three passes, or one resident round,
    // measured 3 to 14 % slower at 1..12 inputs: 180 us = 5.7 TB/s for 1.02 GB at one input).  At two
    // blocks per unit the 64 KB staging of every block is what costs, and one resident round of long
    // blocks wins (217 -> 202 us at sixteen inputs).
    static int resident[DENSE_TOK + 1] = {};                 // blocks per compute unit by staged inputs
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += DENSE_TOK) {
        const uint32_t nt = n_tokens - t0 < (uint32_t)DENSE_TOK ? n_tokens - t0 : (uint32_t)DENSE_TOK;
        const uint32_t lds = nt * (n * 2 + 16);
        int occ = n == 2048 ? resident[nt] : 0;              // cached for the usual width only
        if (occ == 0) {
            NVMAI_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, dense_bf16_gemv_kernel, 256, lds));
            if (occ < 1) occ = 1;
            if (n == 2048) resident[nt] = occ;
        }
        const uint32_t places = (uint32_t)occ * (uint32_t)ctx->compute_units;
        const uint32_t per_block = occ >= 3 ? 1u : (groups + places - 1) / places;
        const dim3 grid((groups + per_block - 1) / per_block);
        dense_bf16_gemv_kernel<<<grid, 256, lds, s>>>(
            w, (const uint16_t*)x + (size_t)t0 * x_stride, x_stride, nt, m, n,
            y ? (uint16_t*)y + (size_t)t0 * y_stride : nullptr, y_f32 ? y_f32 + (size_t)t0 * y_stride : nullptr, y_stride,
            per_block);
    }
    return launch_status();
}
}  // namespace nvmai

namespace {

template <int OP>
int run_elementwise(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* a, const void* b, void* out, uint32_t count) {
    if (!ctx || !a || !b || !out) return NVMAI_ERR_INVALID_ARG;
    if (count == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    if (count >= 4096 && count % 8 == 0 && aligned16(a) && aligned16(out) && (OP == EW_SIGMOID_SCALAR || aligned16(b))) {
        const dim3 grid8((count / 8 + 255) / 256);       // sixteen bytes per thread, the same arithmetic per value
        if (ctx->act == ACT_BF16)
            elementwise8_kernel<ACT_BF16, OP><<<grid8, 256, 0, s>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, count / 8);
        else
            elementwise8_kernel<ACT_FP16, OP><<<grid8, 256, 0, s>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, count / 8);
        return launch_status();
    }
    const dim3 grid((count + 255) / 256);
    if (ctx->act == ACT_BF16)
        elementwise_kernel<ACT_BF16, OP><<<grid, 256, 0, s>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, count);
    else
        elementwise_kernel<ACT_FP16, OP><<<grid, 256, 0, s>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, count);
    return launch_status();
}

}  // namespace

extern "C" int nvmai_hip_silu_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* gate, const void* up,
                                  void* out, uint32_t count) {
    return run_elementwise<EW_SILU_MUL>(ctx, stream, gate, up, out, count);
}

extern "C" int nvmai_hip_sigmoid_gate_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, void* out, const void* gate,
                                          uint32_t count) {
    return run_elementwise<EW_SIGMOID_MUL>(ctx, stream, out, gate, out, count);
}

extern "C" int nvmai_hip_sigmoid_scalar_mul(nvmai_hip_ctx* ctx, nvmai_stream stream, void* y, const void* gate,
                                            uint32_t count) {
    return run_elementwise<EW_SIGMOID_SCALAR>(ctx, stream, y, gate, y, count);
}

extern "C" int nvmai_hip_residual_add(nvmai_hip_ctx* ctx, nvmai_stream stream, void* hidden, const void* delta,
                                      uint32_t count) {
    return run_elementwise<EW_ADD>(ctx, stream, hidden, delta, hidden, count);
}

extern "C" int nvmai_hip_split_q_gate(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* packed, void* q,
                                      void* gate, uint32_t heads, uint32_t dim) {
    if (!ctx || !packed || !q || !gate) return NVMAI_ERR_INVALID_ARG;
    if ((uint64_t)heads * dim > 0x7FFFFFFFull) return NVMAI_ERR_INVALID_ARG;
    if (heads * dim == 0) return NVMAI_OK;
    split_join_rows_kernel<false><<<(heads * dim + 255) / 256, 256, 0, (hipStream_t)stream>>>(
        (uint16_t*)const_cast<void*>(packed), (uint16_t*)q, (uint16_t*)gate, heads, dim);
    return launch_status();
}

extern "C" int nvmai_hip_concat_rows(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* lhs, const void* rhs,
                                     void* out, uint32_t rows, uint32_t dim) {
    if (!ctx || !lhs || !rhs || !out) return NVMAI_ERR_INVALID_ARG;
    if ((uint64_t)rows * dim > 0x7FFFFFFFull) return NVMAI_ERR_INVALID_ARG;
    if (rows * dim == 0) return NVMAI_OK;
    split_join_rows_kernel<true><<<(rows * dim + 255) / 256, 256, 0, (hipStream_t)stream>>>(
        (uint16_t*)out, (uint16_t*)const_cast<void*>(lhs), (uint16_t*)const_cast<void*>(rhs), rows, dim);
    return launch_status();
}

extern "C" int nvmai_hip_embed_lookup(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* table,
                                      const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                                      const uint32_t* token_ids, uint32_t token_id, uint32_t n_tokens, void* out,
                                      uint32_t out_stride, uint32_t d, uint32_t vocab, float out_scale) {
    if (!ctx || !table || !scales || !biases || !out) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (d == 0 || d % NVMAI_GROUP || out_stride < d) return NVMAI_ERR_INVALID_ARG;
    if (n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((d / 8 + 255) / 256, n_tokens);
    if (ctx->act == ACT_BF16)
        embed_lookup_kernel<ACT_BF16><<<grid, 256, 0, s>>>(table, scales, biases, bits, token_ids, token_id, (uint16_t*)out, out_stride, d, vocab, out_scale);
    else
        embed_lookup_kernel<ACT_FP16><<<grid, 256, 0, s>>>(table, scales, biases, bits, token_ids, token_id, (uint16_t*)out, out_stride, d, vocab, out_scale);
    return launch_status();
}

namespace {

template <int ACT, int BITS>
void launch_lm_head(const LmHeadParams& p, uint32_t cpl, dim3 grid, hipStream_t s) {
    const size_t lds = ((size_t)p.d + 16) * 4 + (size_t)p.d * 4;   // floats, block results, two 16-bit rows
    if (cpl <= 1) lm_head_greedy_kernel<ACT, BITS, 1><<<grid, 256, lds, s>>>(p);
    else if (cpl <= 2) lm_head_greedy_kernel<ACT, BITS, 2><<<grid, 256, lds, s>>>(p);
    else lm_head_greedy_kernel<ACT, BITS, 4><<<grid, 256, lds, s>>>(p);
}

}  // namespace

extern "C" int nvmai_hip_lm_head_greedy(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* hidden,
                                        uint32_t hidden_stride, uint32_t n_tokens, const uint16_t* norm_weight,
                                        const uint8_t* weights, const uint16_t* scales, const uint16_t* biases,
                                        uint32_t bits, uint32_t* out_tokens, uint32_t d, uint32_t vocab,
                                        float rms_eps) {
    if (!ctx || !hidden || !weights || !scales || !biases || !out_tokens) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (d == 0 || d % NVMAI_GROUP || hidden_stride < d || vocab == 0) return NVMAI_ERR_INVALID_ARG;   // LMHeadChainInt4.swift:76-77
    const uint32_t chunks = d * bits / 128;        // d is a multiple of 64: whole 16-byte chunks
    const uint32_t cpl = (chunks + 31) / 32;
    if (cpl > 4) return NVMAI_ERR_UNSUPPORTED;     // rows of at most 2048 bytes
    if (!aligned16(weights)) return NVMAI_ERR_ALIGNMENT;
    if (n_tokens == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t n_blocks = (vocab + LMH_ROWS - 1) / LMH_ROWS;
    int rc = ws_begin(ctx, stream, ws_round((size_t)n_tokens * n_blocks * sizeof(float2)));
    if (rc) return rc;
    LmHeadParams p{};
    p.hidden = (const uint16_t*)hidden; p.hidden_stride = hidden_stride; p.norm_weight = norm_weight;
    p.weights = weights; p.scales = scales; p.biases = biases; p.d = d; p.vocab = vocab; p.eps = rms_eps;
    p.summaries = ws_take<float2>(ctx, (size_t)n_tokens * n_blocks);
    const dim3 grid(n_blocks, n_tokens);
    if (ctx->act == ACT_BF16) {
        if (bits == 8) launch_lm_head<ACT_BF16, 8>(p, cpl, grid, s); else launch_lm_head<ACT_BF16, 4>(p, cpl, grid, s);
    } else {
        if (bits == 8) launch_lm_head<ACT_FP16, 8>(p, cpl, grid, s); else launch_lm_head<ACT_FP16, 4>(p, cpl, grid, s);
    }
    lm_head_reduce_kernel<<<n_tokens, 256, 0, s>>>(p.summaries, n_blocks, out_tokens);
    return launch_status();
}
