// Entry points: gated-DeltaNet linear attention (conv + q / k norm, delta rule + gated output norm)
// and the fused input projections of an attention block.
#include "ctx.hpp"
#include "gdn_kernels.hpp"
#include "gdn_chunk_kernels.hpp"
#include "gdn_wy_kernels.hpp"

using namespace nvmai;

namespace {

int check_gdn(const nvmai_gdn_config* c, uint32_t rows, uint32_t batch) {
    if (!c || rows == 0 || batch == 0) return NVMAI_ERR_INVALID_ARG;
    // GDN.init preconditions (GDN.swift:38-45)
    if (c->key_head_dim == 0 || c->key_head_dim % 32 || c->value_head_dim == 0 || c->value_head_dim % 4 ||
        c->num_k_heads == 0 || c->num_v_heads == 0 || c->num_v_heads % c->num_k_heads)
        return NVMAI_ERR_INVALID_ARG;
    if (c->conv_kernel_size == 0 || c->conv_kernel_size > GDN_MAX_TAPS) return NVMAI_ERR_UNSUPPORTED;
    return NVMAI_OK;
}

GdnShape shape_of(const nvmai_gdn_config* c, uint32_t rows, uint32_t batch) {
    return GdnShape{c->num_k_heads, c->num_v_heads, c->key_head_dim, c->value_head_dim, c->conv_kernel_size, rows, batch};
}

// From this many rows per sequence on a call takes the kernels that keep only the recurrence
// sequential (two or three launches instead of one or two, so not for a handful of rows).
constexpr uint32_t GDN_ROWS_PARALLEL_FROM = 8;

// From this many rows per sequence on the recurrence of a 128 x 128 head runs sixteen rows at a time on
// the matrix cores (one or two launches more, and workspace per head and chunk: launch_delta_chunked).
constexpr uint32_t GDN_CHUNKED_FROM = 64;

// The gated norm over the rows the recurrence left in out: heads of 128 values in 16-byte pieces where
// the rows allow it (same bits), one value per thread otherwise.  (rows + 1) / 2 <= 65535 is the caller's.
template <int ACT>
void launch_gated_norm_rows(const GdnDeltaParams& p, hipStream_t s) {
    const uint64_t units = (uint64_t)p.sh.batch * p.sh.rows * p.sh.v_heads;
    if (p.sh.dv == 128 && units < (1ull << 31) && aligned16(p.out) && p.out_stride % 8 == 0 && aligned16(p.z) &&
        p.z_stride % 8 == 0 && aligned16(p.norm_w)) {
        gdn_gated_norm_rows128_kernel<ACT><<<dim3((uint32_t)((units + 15) / 16)), 256, 0, s>>>(
            p.out, p.out_stride, p.z, p.z_stride, p.norm_w, p.sh, (uint32_t)units);
        return;
    }
    const dim3 ngrid(p.sh.v_heads, p.sh.batch, (p.sh.rows + 1) / 2);
    gdn_gated_norm_rows_kernel<ACT><<<ngrid, 256, 0, s>>>(p.out, p.out_stride, p.z, p.z_stride, p.norm_w, p.sh);
}

// Returns 1 = launched, 0 = not a shape or alignment this form takes (the caller goes on to the row-by-row
// kernels), or a negative status: the workspace could not be had -- in particular NVMAI_ERR_SCRATCH when it
// would have to grow while the stream is being captured.  That is handed back to the caller instead of taking
// the other kernels silently: their summation order differs, so a captured call would not give the bits of
// the eager one.  Reserve (sizeof(GdnChunkPrep) = 2,304 bytes, and with BF16 activations sizeof(GdnChunkWY) = 8,192
// more) * batch * value heads * ceil(rows / 16), and with BF16 activations sizeof(GdnChunkKT) = 4,096 * batch * key
// heads * ceil(rows / 16), with nvmai_hip_ctx_reserve (or run the same call eagerly once) before capturing.
template <int ACT, int DK, int DV>
int launch_delta_chunked(nvmai_hip_ctx* ctx, const GdnDeltaParams& p, bool state_bf16, hipStream_t s) {
    if (DK != 128 || DV != 128) return 0;
    const uint32_t nchunks = (p.sh.rows + 15) / 16;
    const size_t count = (size_t)p.sh.batch * p.sh.v_heads * nchunks;
    if (!ctx || nchunks > 65535 || p.sh.batch > 65535 || (p.sh.rows + 1) / 2 > 65535 || !aligned16(p.conv_out) || p.conv_stride % 8 ||
        (!state_bf16 && !aligned16(p.state)) || (reinterpret_cast<uintptr_t>(p.state) & 7u))
        return 0;
    // BF16 activations: the chain on the 16-bit matrix instructions from operands prepared per chunk
    // (8,192 bytes more per (sequence, value head, chunk) and 4,096 per (sequence, key head, chunk))
    const bool wy_form = ACT == ACT_BF16;
    const size_t count_k = (size_t)p.sh.batch * p.sh.k_heads * nchunks;
    const size_t wy_bytes = wy_form ? ws_round(count * sizeof(GdnChunkWY)) + ws_round(count_k * sizeof(GdnChunkKT)) : 0;
    const int ws_rc = ws_begin(ctx, (nvmai_stream)s, ws_round(count * sizeof(GdnChunkPrep)) + wy_bytes);
    if (ws_rc != NVMAI_OK) return ws_rc;
    GdnChunkPrep* prep = ws_take<GdnChunkPrep>(ctx, count);
    const dim3 cgrid(p.sh.v_heads, p.sh.batch, 128 / 16);
    if (wy_form) {
        GdnChunkWY* wy = ws_take<GdnChunkWY>(ctx, count);
        GdnChunkKT* kts = ws_take<GdnChunkKT>(ctx, count_k);
        gdn_wy_prep_kernel<<<dim3(nchunks, p.sh.v_heads, p.sh.batch), 64, 0, s>>>(p, prep, wy, kts, nchunks);
        if (state_bf16) gdn_wy_delta_kernel<true><<<cgrid, 64 * GDN_WY_WAVES, 0, s>>>(p, prep, wy, kts, nchunks);
        else gdn_wy_delta_kernel<false><<<cgrid, 64 * GDN_WY_WAVES, 0, s>>>(p, prep, wy, kts, nchunks);
    } else {
        gdn_chunk_prep_kernel<ACT, 128><<<dim3(nchunks, p.sh.v_heads, p.sh.batch), 64, 0, s>>>(p, prep, nchunks);
        if (state_bf16) gdn_chunk_delta_kernel<ACT, 128, 128, true><<<cgrid, 64 * GDN_CHUNK_WAVES, 0, s>>>(p, prep, nchunks);
        else gdn_chunk_delta_kernel<ACT, 128, 128, false><<<cgrid, 64 * GDN_CHUNK_WAVES, 0, s>>>(p, prep, nchunks);
    }
    launch_gated_norm_rows<ACT>(p, s);
    return 1;
}

template <int ACT, int DK, int DV>
int launch_delta(nvmai_hip_ctx* ctx, const GdnDeltaParams& p, bool state_bf16, hipStream_t s) {
    const dim3 grid(p.sh.v_heads, p.sh.batch);
    if (p.sh.rows >= GDN_CHUNKED_FROM) {
        const int rc = launch_delta_chunked<ACT, DK, DV>(ctx, p, state_bf16, s);
        if (rc != 0) return rc < 0 ? rc : NVMAI_OK;
    }
    if (p.sh.rows >= GDN_ROWS_PARALLEL_FROM && (p.sh.rows + 1) / 2 <= 65535 && aligned16(p.conv_out) && p.conv_stride % 8 == 0) {
        const dim3 rgrid(p.sh.v_heads, p.sh.batch, DV / 16);      // one group of sixteen state rows per block
        if (state_bf16) gdn_delta_rows_kernel<ACT, DK, DV, true, 1><<<rgrid, 256, 0, s>>>(p);
        else gdn_delta_rows_kernel<ACT, DK, DV, false, 1><<<rgrid, 256, 0, s>>>(p);
        launch_gated_norm_rows<ACT>(p, s);
        return NVMAI_OK;
    }
    if (DK == 128 && DV == 128 && aligned16(p.state)) {       // the production head, state rows in 16-byte pieces
        if (state_bf16) gdn_delta_gated_kernel<ACT, DK, DV, true, DK == 128><<<grid, 256, 0, s>>>(p);
        else gdn_delta_gated_kernel<ACT, DK, DV, false, DK == 128><<<grid, 256, 0, s>>>(p);
        return NVMAI_OK;
    }
    if (state_bf16) gdn_delta_gated_kernel<ACT, DK, DV, true><<<grid, 256, 0, s>>>(p);
    else gdn_delta_gated_kernel<ACT, DK, DV, false><<<grid, 256, 0, s>>>(p);
    return NVMAI_OK;
}

template <int ACT>
int launch_delta_shape(nvmai_hip_ctx* ctx, const GdnDeltaParams& p, bool state_bf16, hipStream_t s) {
    const uint32_t dk = p.sh.dk, dv = p.sh.dv;
    if (dk == 128 && dv == 128) return launch_delta<ACT, 128, 128>(ctx, p, state_bf16, s);
    if (dk == 64 && dv == 64) return launch_delta<ACT, 64, 64>(ctx, p, state_bf16, s);
    if (dk == 32 && dv == 32) return launch_delta<ACT, 32, 32>(ctx, p, state_bf16, s);
    if (dk == 64 && dv == 128) return launch_delta<ACT, 64, 128>(ctx, p, state_bf16, s);
    if (dk == 128 && dv == 64) return launch_delta<ACT, 128, 64>(ctx, p, state_bf16, s);
    return NVMAI_ERR_UNSUPPORTED;
}

}  // namespace

extern "C" int nvmai_hip_gdn_conv_norm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                                       const void* qkv_raw, uint32_t qkv_stride, void* tail, const uint16_t* conv_weight,
                                       void* conv_out, uint32_t conv_out_stride, uint32_t rows, uint32_t batch) {
    if (!ctx || !qkv_raw || !tail || !conv_weight || !conv_out) return NVMAI_ERR_INVALID_ARG;
    int rc = check_gdn(config, rows, batch);
    if (rc) return rc;
    const uint32_t C = 2 * config->num_k_heads * config->key_head_dim + config->num_v_heads * config->value_head_dim;
    if (qkv_stride < C || conv_out_stride < C) return NVMAI_ERR_INVALID_ARG;
    const GdnShape sh = shape_of(config, rows, batch);
    const dim3 grid(2 * sh.k_heads + sh.v_heads, batch);
    hipStream_t s = (hipStream_t)stream;
    if (rows >= GDN_ROWS_PARALLEL_FROM && sh.dk <= 128 && sh.dv <= 128 && (rows + 1) / 2 <= 65535) {
        // a chunk of rows: thirty-two rows of a head segment per block, then the tail in a launch of its own
        const dim3 rgrid(2 * sh.k_heads + sh.v_heads, batch, (rows + GDN_CONV_ROWS_PER_BLOCK - 1) / GDN_CONV_ROWS_PER_BLOCK);
        const bool pieces = sh.taps == 4 && sh.dk % 8 == 0 && sh.dv % 8 == 0 && qkv_stride % 8 == 0 && conv_out_stride % 8 == 0 &&
                            aligned16(qkv_raw) && aligned16(tail) && aligned16(conv_weight) && aligned16(conv_out);
        if (pieces) {
            // rows in 16-byte pieces: eight rows of a head segment per sixteen lanes
            const dim3 pgrid(2 * sh.k_heads + sh.v_heads, batch, (rows + GDN_CONV8_ROWS_PER_BLOCK - 1) / GDN_CONV8_ROWS_PER_BLOCK);
            if (ctx->act == ACT_BF16)
                gdn_conv_norm_rows8_kernel<ACT_BF16><<<pgrid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (const uint16_t*)tail,
                                                                          conv_weight, (uint16_t*)conv_out, conv_out_stride, sh);
            else
                gdn_conv_norm_rows8_kernel<ACT_FP16><<<pgrid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (const uint16_t*)tail,
                                                                          conv_weight, (uint16_t*)conv_out, conv_out_stride, sh);
        } else if (ctx->act == ACT_BF16)
            gdn_conv_norm_rows_kernel<ACT_BF16><<<rgrid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (const uint16_t*)tail,
                                                                     conv_weight, (uint16_t*)conv_out, conv_out_stride, sh);
        else
            gdn_conv_norm_rows_kernel<ACT_FP16><<<rgrid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (const uint16_t*)tail,
                                                                     conv_weight, (uint16_t*)conv_out, conv_out_stride, sh);
        if (sh.taps > 1)
            gdn_tail_update_kernel<<<dim3((C + 255) / 256, batch), 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride,
                                                                               (uint16_t*)tail, sh);
        return launch_status();
    }
    if (ctx->act == ACT_BF16)
        gdn_conv_norm_kernel<ACT_BF16><<<grid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (uint16_t*)tail, conv_weight,
                                                            (uint16_t*)conv_out, conv_out_stride, sh);
    else
        gdn_conv_norm_kernel<ACT_FP16><<<grid, 256, 0, s>>>((const uint16_t*)qkv_raw, qkv_stride, (uint16_t*)tail, conv_weight,
                                                            (uint16_t*)conv_out, conv_out_stride, sh);
    return launch_status();
}

extern "C" int nvmai_hip_gdn_delta_gated_norm(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                                              const void* conv_out, uint32_t conv_out_stride, const void* a_proj,
                                              const void* b_proj, uint32_t ab_stride, const uint16_t* a_log,
                                              const uint16_t* dt_bias, void* state, int state_is_bf16, const void* z,
                                              uint32_t z_stride, const uint16_t* norm_weight, void* out,
                                              uint32_t out_stride, uint32_t rows, uint32_t batch) {
    if (!ctx || !conv_out || !a_proj || !b_proj || !a_log || !dt_bias || !state || !z || !norm_weight || !out)
        return NVMAI_ERR_INVALID_ARG;
    int rc = check_gdn(config, rows, batch);
    if (rc) return rc;
    const uint32_t C = 2 * config->num_k_heads * config->key_head_dim + config->num_v_heads * config->value_head_dim;
    const uint32_t vd = config->num_v_heads * config->value_head_dim;
    if (conv_out_stride < C || ab_stride < config->num_v_heads || z_stride < vd || out_stride < vd) return NVMAI_ERR_INVALID_ARG;
    GdnDeltaParams p{};
    p.conv_out = (const uint16_t*)conv_out; p.conv_stride = conv_out_stride;
    p.a_proj = (const uint16_t*)a_proj; p.b_proj = (const uint16_t*)b_proj; p.ab_stride = ab_stride;
    p.a_log = a_log; p.dt_bias = dt_bias; p.state = state;
    p.z = (const uint16_t*)z; p.z_stride = z_stride; p.norm_w = norm_weight;
    p.out = (uint16_t*)out; p.out_stride = out_stride;
    p.sh = shape_of(config, rows, batch);
    hipStream_t s = (hipStream_t)stream;
    rc = ctx->act == ACT_BF16 ? launch_delta_shape<ACT_BF16>(ctx, p, state_is_bf16 != 0, s)
                              : launch_delta_shape<ACT_FP16>(ctx, p, state_is_bf16 != 0, s);
    if (rc) return rc;
    return launch_status();
}

namespace {
template <int ACT, int DK, int DV>
bool launch_decode_fused(const GdnDecodeParams& p, uint32_t ratio, bool state_bf16, hipStream_t s) {
    const dim3 grid(p.d.sh.k_heads, p.d.sh.batch);
#define NVMAI_GDN_FUSED(R)                                                                             \
    do {                                                                                               \
        if (state_bf16) gdn_decode_fused_kernel<ACT, DK, DV, R, true><<<grid, 256 * R, 0, s>>>(p);      \
        else gdn_decode_fused_kernel<ACT, DK, DV, R, false><<<grid, 256 * R, 0, s>>>(p);                \
        return true;                                                                                   \
    } while (0)
    if (ratio == 1) NVMAI_GDN_FUSED(1);
    if (ratio == 2) NVMAI_GDN_FUSED(2);
#undef NVMAI_GDN_FUSED
    return false;
}

template <int ACT>
bool launch_decode_fused_shape(const GdnDecodeParams& p, uint32_t ratio, bool state_bf16, hipStream_t s) {
    const uint32_t dk = p.d.sh.dk, dv = p.d.sh.dv;
    if (dk == 128 && dv == 128) return launch_decode_fused<ACT, 128, 128>(p, ratio, state_bf16, s);
    if (dk == 32 && dv == 32) return launch_decode_fused<ACT, 32, 32>(p, ratio, state_bf16, s);
    return false;
}
}  // namespace

extern "C" int nvmai_hip_gdn_decode_step(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gdn_config* config,
                                         const void* qkv_raw, uint32_t qkv_stride, void* tail, const uint16_t* conv_weight,
                                         void* conv_scratch, uint32_t conv_scratch_stride, const void* a_proj,
                                         const void* b_proj, uint32_t ab_stride, const uint16_t* a_log,
                                         const uint16_t* dt_bias, void* state, int state_is_bf16, const void* z,
                                         uint32_t z_stride, const uint16_t* norm_weight, void* out, uint32_t out_stride,
                                         uint32_t batch) {
    if (!ctx || !qkv_raw || !tail || !conv_weight || !a_proj || !b_proj || !a_log || !dt_bias || !state || !z ||
        !norm_weight || !out)
        return NVMAI_ERR_INVALID_ARG;
    int rc = check_gdn(config, 1, batch);
    if (rc) return rc;
    const uint32_t C = 2 * config->num_k_heads * config->key_head_dim + config->num_v_heads * config->value_head_dim;
    const uint32_t vd = config->num_v_heads * config->value_head_dim;
    if (qkv_stride < C || ab_stride < config->num_v_heads || z_stride < vd || out_stride < vd) return NVMAI_ERR_INVALID_ARG;
    GdnDecodeParams p{};
    p.d.a_proj = (const uint16_t*)a_proj; p.d.b_proj = (const uint16_t*)b_proj; p.d.ab_stride = ab_stride;
    p.d.a_log = a_log; p.d.dt_bias = dt_bias; p.d.state = state;
    p.d.z = (const uint16_t*)z; p.d.z_stride = z_stride; p.d.norm_w = norm_weight;
    p.d.out = (uint16_t*)out; p.d.out_stride = out_stride;
    p.d.sh = shape_of(config, 1, batch);
    p.qkv_raw = (const uint16_t*)qkv_raw; p.qkv_stride = qkv_stride; p.tail = (uint16_t*)tail; p.conv_w = conv_weight;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t ratio = config->num_v_heads / config->num_k_heads;
    const bool fused = ctx->act == ACT_BF16 ? launch_decode_fused_shape<ACT_BF16>(p, ratio, state_is_bf16 != 0, s)
                                            : launch_decode_fused_shape<ACT_FP16>(p, ratio, state_is_bf16 != 0, s);
    if (fused) return launch_status();
    // a shape without a fused instantiation: the two kernels one after the other through the scratch rows
    if (!conv_scratch || conv_scratch_stride < C) return NVMAI_ERR_UNSUPPORTED;
    rc = nvmai_hip_gdn_conv_norm(ctx, stream, config, qkv_raw, qkv_stride, tail, conv_weight, conv_scratch,
                                 conv_scratch_stride, 1, batch);
    if (rc) return rc;
    return nvmai_hip_gdn_delta_gated_norm(ctx, stream, config, conv_scratch, conv_scratch_stride, a_proj, b_proj, ab_stride,
                                          a_log, dt_bias, state, state_is_bf16, z, z_stride, norm_weight, out, out_stride,
                                          1, batch);
}

// One GEMV launch over the concatenated rows of several matrices when they lie back to back in
// memory (codes, scales and biases each, and the outputs), one launch per matrix otherwise.
extern "C" int nvmai_hip_affine_gemv_fused(nvmai_hip_ctx* ctx, nvmai_stream stream, const nvmai_gemv_part* parts,
                                           uint32_t n_parts, uint32_t bits, const void* x, uint32_t x_stride,
                                           uint32_t n_tokens, uint32_t n) {
    if (!ctx || !parts || n_parts == 0 || !x) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || n % NVMAI_GROUP) return NVMAI_ERR_INVALID_ARG;
    const uint64_t row_bytes = (uint64_t)n * bits / 8, meta_bytes = (uint64_t)(n / NVMAI_GROUP) * 2;
    bool adjacent = n_tokens == 1;        // rows of one input are contiguous in the output; more inputs need a common stride
    uint32_t total = 0;
    for (uint32_t i = 0; i < n_parts; ++i) {
        const nvmai_gemv_part& a = parts[i];
        if (!a.weights || !a.scales || !a.biases || !a.y || a.y_stride < a.rows) return NVMAI_ERR_INVALID_ARG;
        total += a.rows;
        if (i + 1 < n_parts) {
            const nvmai_gemv_part& b = parts[i + 1];
            adjacent = adjacent && b.weights == a.weights + a.rows * row_bytes &&
                       (const uint8_t*)b.scales == (const uint8_t*)a.scales + a.rows * meta_bytes &&
                       (const uint8_t*)b.biases == (const uint8_t*)a.biases + a.rows * meta_bytes &&
                       (const uint8_t*)b.y == (const uint8_t*)a.y + (size_t)a.rows * 2;
        }
    }
    if (adjacent)
        return nvmai_hip_affine_gemv(ctx, stream, parts[0].weights, parts[0].scales, parts[0].biases, bits, x, x_stride,
                                     n_tokens, total, n, parts[0].y, nullptr, total);
    for (uint32_t i = 0; i < n_parts; ++i) {
        const nvmai_gemv_part& a = parts[i];
        if (a.rows == 0) continue;
        const int rc = nvmai_hip_affine_gemv(ctx, stream, a.weights, a.scales, a.biases, bits, x, x_stride, n_tokens,
                                             a.rows, n, a.y, nullptr, a.y_stride);
        if (rc) return rc;
    }
    return NVMAI_OK;
}
