// Entry points: KV row layout, quantize-on-write, partial RoPE, GQA decode attention.
#include <cmath>

#include "attn_kernels.hpp"
#include "attn_prefill_kernels.hpp"
#include "ctx.hpp"

using namespace nvmai;

extern "C" int nvmai_kv_row_layout(uint32_t elements, uint32_t bits, uint32_t* stride, uint32_t* value_bytes) {
    if (!stride || !value_bytes || elements == 0) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8 && bits != 16) return NVMAI_ERR_UNSUPPORTED;
    if (bits == 16) { *stride = elements * 2; *value_bytes = elements * 2; return NVMAI_OK; }
    const uint32_t packed = (elements * bits + 7) / 8;
    const uint32_t aligned = (packed + 1) & ~1u;
    const uint32_t groups = (elements + 63) / 64;
    *stride = aligned + groups * 4;
    *value_bytes = aligned;
    return NVMAI_OK;
}

extern "C" int nvmai_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                                              uint32_t kv_start, int prefer_gqa_swa, uint32_t* effective_length,
                                              uint32_t* num_chunks, uint32_t* chunk_length,
                                              uint32_t* partial_threadgroups) {
    if (!num_kv_heads || num_q_heads % num_kv_heads || !effective_length || !num_chunks || !chunk_length ||
        !partial_threadgroups)
        return NVMAI_ERR_INVALID_ARG;
    const long q_per_kv = num_q_heads / num_kv_heads;
    const bool use_gqa = prefer_gqa_swa && q_per_kv <= 2;
    const long eff = (long)seq_len - (long)kv_start, e1 = eff > 1 ? eff : 1;
    long base = use_gqa ? 8 : 16;                    // Attention.swift:53-54
    if (e1 < base) base = e1;
    long nc = base;
    if (use_gqa) { long alt = base * q_per_kv; if (alt > 64) alt = 64; if (alt > nc) nc = alt; }
    *effective_length = (uint32_t)eff;
    *num_chunks = (uint32_t)nc;
    *chunk_length = (uint32_t)((e1 + nc - 1) / nc);
    *partial_threadgroups = (uint32_t)((use_gqa ? num_kv_heads : num_q_heads) * nc);
    return NVMAI_OK;
}

namespace {
int check_view(const nvmai_kv_view* v, uint32_t elements) {
    if (!v || !v->base) return NVMAI_ERR_INVALID_ARG;
    if (v->bits != 4 && v->bits != 8 && v->bits != 16) return NVMAI_ERR_UNSUPPORTED;
    if (v->group_size != 64) return NVMAI_ERR_UNSUPPORTED;
    uint32_t stride = 0, vb = 0;
    if (nvmai_kv_row_layout(elements, v->bits, &stride, &vb) != NVMAI_OK) return NVMAI_ERR_INVALID_ARG;
    if (v->value_bytes != vb || v->stride < stride || (v->stride & 1u)) return NVMAI_ERR_INVALID_ARG;
    return NVMAI_OK;
}
}  // namespace

extern "C" int nvmai_hip_kv_quantize_affine(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* source,
                                            uint32_t source_stride, const nvmai_kv_view* dst,
                                            uint32_t token_count, uint32_t element_count) {
    if (!ctx || !source || element_count == 0 || source_stride < element_count) return NVMAI_ERR_INVALID_ARG;
    int rc = check_view(dst, element_count);
    if (rc) return rc;
    if (dst->bits == 16) return NVMAI_ERR_UNSUPPORTED;        // "KV quantizer requires 4-bit or 8-bit destination"
    if (token_count == 0) return NVMAI_ERR_INVALID_ARG;       // KVCacheQuantizer.swift:22
    KvFormat f{dst->bits, dst->stride, dst->value_bytes, element_count};
    ProfScope ps(ctx, NVMAI_PROF_KV_QUANT, (hipStream_t)stream);
    if (element_count % 64 == 0 && aligned16(source) && source_stride % 8 == 0 &&
        (reinterpret_cast<uintptr_t>(dst->base) & 7u) == 0 && dst->stride % 8 == 0) {
        const uint64_t threads = (uint64_t)token_count * (element_count / 8);
        dim3 vgrid((uint32_t)((threads + 255) / 256));
        hipStream_t s = (hipStream_t)stream;
#define NVMAI_KVQ(ACT, BITS) \
    kv_quantize_vec_kernel<ACT, BITS><<<vgrid, 256, 0, s>>>(source, source_stride, (uint8_t*)dst->base, f, token_count)
        if (ctx->act == ACT_BF16) { if (dst->bits == 8) NVMAI_KVQ(ACT_BF16, 8); else NVMAI_KVQ(ACT_BF16, 4); }
        else { if (dst->bits == 8) NVMAI_KVQ(ACT_FP16, 8); else NVMAI_KVQ(ACT_FP16, 4); }
#undef NVMAI_KVQ
        return launch_status();
    }
    const uint64_t waves = (uint64_t)token_count * ((element_count + 63) / 64);
    dim3 grid((uint32_t)((waves + 3) / 4));
    if (ctx->act == ACT_BF16) kv_quantize_kernel<ACT_BF16><<<grid, 256, 0, (hipStream_t)stream>>>(source, source_stride, (uint8_t*)dst->base, f, token_count);
    else kv_quantize_kernel<ACT_FP16><<<grid, 256, 0, (hipStream_t)stream>>>(source, source_stride, (uint8_t*)dst->base, f, token_count);
    return launch_status();
}

extern "C" int nvmai_hip_rope_neox_subdim(nvmai_hip_ctx* ctx, nvmai_stream stream, void* data, uint32_t tokens,
                                          uint32_t heads, uint32_t head_dim, uint32_t rotary_dim,
                                          const uint32_t* positions, uint32_t position, float theta) {
    if (!ctx || !data || rotary_dim > head_dim || (rotary_dim & 1u) || heads == 0 || head_dim == 0)
        return NVMAI_ERR_INVALID_ARG;
    const uint64_t n = (uint64_t)tokens * heads * (rotary_dim / 2);
    if (n == 0) return NVMAI_OK;
    dim3 grid((uint32_t)((n + 255) / 256));
    if (ctx->act == ACT_BF16) rope_neox_subdim_kernel<ACT_BF16><<<grid, 256, 0, (hipStream_t)stream>>>(data, tokens, heads, head_dim, rotary_dim, positions, position, theta);
    else rope_neox_subdim_kernel<ACT_FP16><<<grid, 256, 0, (hipStream_t)stream>>>(data, tokens, heads, head_dim, rotary_dim, positions, position, theta);
    return launch_status();
}

namespace {
// Shared by the decode, ragged decode and causal prefill entry points.  p holds the problem (q, out
// and their strides, the views' format, the per-sequence range rule, batch, heads); max_len is the
// longest key range any block may have to walk, pack_ok says that every sequence reads the same
// cache so several of them may share a block's K/V reads.
int run_attention(nvmai_hip_ctx* ctx, nvmai_stream stream, AttnParams p, const nvmai_kv_view* k,
                  const nvmai_kv_view* v, uint32_t max_len, bool pack_ok) {
    hipStream_t s = (hipStream_t)stream;
    const uint32_t qpk = p.num_q_heads / p.num_kv_heads;
    const bool fast = p.head_dim == ATTN_HD && (k->bits == 4 || k->bits == 8) && qpk <= 16 && p.ring == 0 &&
                      aligned16(k->base) && aligned16(v->base) && (k->stride % 16 == 0) &&
                      (p.kv_batch_stride % 16 == 0) && aligned16(p.q) && (p.q_stride % 8 == 0) &&
                      (uint64_t)p.seq_len * k->stride < (1ull << 32);      // 32-bit row offsets in the kernel
    p.cols_q = (fast && pack_ok) ? 16 / qpk : 1;
    const uint32_t seq_blocks = (p.batch + p.cols_q - 1) / p.cols_q;
    if (p.cols_q > 1) max_len = max_len + p.cols_q - 1 < p.seq_len ? max_len + p.cols_q - 1 : p.seq_len;
    // Chunking: enough blocks to fill the device, chunks a multiple of the 32-token step.
    const uint64_t units = fast ? (uint64_t)seq_blocks * p.num_kv_heads : (uint64_t)p.batch * p.num_q_heads;
    const uint32_t len = max_len;
    // blocks aimed at: two per compute unit, except the 8-bit matrix-core kernel, which is bound by bytes
    // and does better with one block per unit and half the partial rows to write and merge (32K x 1:
    // 20.2 -> 17.8 us, 128K x 1: 40.9 -> 35.1, 32K x 8: 62.2 -> 58.3; the 4-bit kernel, bound by its vector
    // work, loses with one: 128K x 8 136 -> 165 us)
    const uint32_t tgt = (fast && k->bits == 8) ? 256u : 512u;
    uint32_t nc = units >= tgt ? 1 : (uint32_t)((tgt + units - 1) / units);
    const uint32_t max_nc = (len + 127) / 128 ? (len + 127) / 128 : 1;
    if (nc > max_nc) nc = max_nc;
    if (nc < 1) nc = 1;
    uint32_t chunk_len = ((len > 0 ? len : 1) + nc - 1) / nc;
    chunk_len = (chunk_len + 31) & ~31u;
    nc = ((len > 0 ? len : 1) + chunk_len - 1) / chunk_len;
    if (nc > ATTN_MAX_CHUNKS) return NVMAI_ERR_UNSUPPORTED;      // cannot happen: nc <= 512 by construction
    const size_t heads_total = (size_t)p.batch * p.num_q_heads;
    // one chunk: the partial kernel writes the rows itself (the matrix-core one in 8-byte pieces)
    // (a gated call keeps the combine launch: the gate is applied where the rows are written)
    p.direct = nc == 1 && !p.gate && (!fast || ((reinterpret_cast<uintptr_t>(p.out) & 7u) == 0 && p.out_stride % 4 == 0));
    p.num_chunks = nc; p.chunk_len = chunk_len;
    if (!p.direct) {
        const int rc = ws_begin(ctx, stream, 2 * ws_round(heads_total * nc * 4) + ws_round(heads_total * nc * p.head_dim * 4));
        if (rc) return rc;
        p.m_part = ws_take<float>(ctx, heads_total * nc);
        p.d_part = ws_take<float>(ctx, heads_total * nc);
        p.o_part = ws_take<float>(ctx, heads_total * nc * p.head_dim);
    }
    {
        ProfScope ps(ctx, NVMAI_PROF_ATTN_PARTIAL, s);
        if (fast) {
            dim3 grid(seq_blocks * p.num_kv_heads * nc);
#define NVMAI_ATTN(ACT, BITS) attn_partial_mfma_kernel<ACT, BITS><<<grid, 256, 0, s>>>(p)
            if (ctx->act == ACT_BF16) { if (k->bits == 8) NVMAI_ATTN(ACT_BF16, 8); else NVMAI_ATTN(ACT_BF16, 4); }
            else { if (k->bits == 8) NVMAI_ATTN(ACT_FP16, 8); else NVMAI_ATTN(ACT_FP16, 4); }
#undef NVMAI_ATTN
        } else {
            dim3 grid(p.batch * p.num_q_heads * nc);
            if (ctx->act == ACT_BF16) attn_partial_generic_kernel<ACT_BF16><<<grid, 256, 0, s>>>(p);
            else attn_partial_generic_kernel<ACT_FP16><<<grid, 256, 0, s>>>(p);
        }
    }
    if (!p.direct) {
        ProfScope ps(ctx, NVMAI_PROF_ATTN_COMBINE, s);
        const dim3 cgrid((uint32_t)heads_total, (p.head_dim + 63) / 64);
        if (ctx->act == ACT_BF16) attn_combine_kernel<ACT_BF16><<<cgrid, 256, 0, s>>>(p);
        else attn_combine_kernel<ACT_FP16><<<cgrid, 256, 0, s>>>(p);
    }
    return launch_status();
}

// Argument checks common to the three entry points; fills the shape and format fields of p.
int attention_setup(nvmai_hip_ctx* ctx, const void* q, const nvmai_kv_view* k, const nvmai_kv_view* v, void* out,
                    uint32_t batch, uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads, float scale,
                    AttnParams& p) {
    if (!ctx || !q || !out || batch == 0 || head_dim == 0 || num_kv_heads == 0 || num_q_heads == 0) return NVMAI_ERR_INVALID_ARG;
    if (num_q_heads % num_kv_heads) return NVMAI_ERR_INVALID_ARG;      // Attention.swift:221-222
    if (head_dim > 512) return NVMAI_ERR_INVALID_ARG;                  // Attention.swift:223-224
    const uint32_t elements = num_kv_heads * head_dim;
    int rc = check_view(k, elements);
    if (rc) return rc;
    rc = check_view(v, elements);
    if (rc) return rc;
    if (k->bits != v->bits || k->stride != v->stride) return NVMAI_ERR_INVALID_ARG;
    p = AttnParams{};
    p.q = q; p.out = out; p.k = (const uint8_t*)k->base; p.v = (const uint8_t*)v->base;
    p.f = KvFormat{k->bits, k->stride, k->value_bytes, elements};
    p.head_dim = head_dim; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.batch = batch;
    p.q_stride = p.out_stride = num_q_heads * head_dim;
    p.scale = scale > 0.0f ? scale : 1.0f / std::sqrt((float)head_dim);
    return NVMAI_OK;
}
}  // namespace

extern "C" int nvmai_hip_attention_decode(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                          const nvmai_kv_view* k, const nvmai_kv_view* v,
                                          uint64_t kv_batch_stride, void* out, uint32_t batch,
                                          uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                          uint32_t seq_len, uint32_t kv_start, float scale) {
    AttnParams p;
    const int rc = attention_setup(ctx, q, k, v, out, batch, head_dim, num_q_heads, num_kv_heads, scale, p);
    if (rc) return rc;
    if (kv_start > seq_len) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(q)) return NVMAI_ERR_ALIGNMENT;
    p.kv_batch_stride = kv_batch_stride;
    p.seq_len = seq_len; p.kv_start = kv_start;
    return run_attention(ctx, stream, p, k, v, seq_len - kv_start, false);
}

extern "C" int nvmai_hip_attention_decode_gated(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                                const nvmai_kv_view* k, const nvmai_kv_view* v,
                                                uint64_t kv_batch_stride, void* out, const void* gate,
                                                uint32_t gate_stride, uint32_t batch, uint32_t head_dim,
                                                uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                                                uint32_t kv_start, float scale) {
    AttnParams p;
    const int rc = attention_setup(ctx, q, k, v, out, batch, head_dim, num_q_heads, num_kv_heads, scale, p);
    if (rc) return rc;
    if (kv_start > seq_len || !gate || gate_stride < num_q_heads * head_dim) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(q)) return NVMAI_ERR_ALIGNMENT;
    p.kv_batch_stride = kv_batch_stride;
    p.seq_len = seq_len; p.kv_start = kv_start;
    p.gate = (const uint16_t*)gate; p.gate_stride = gate_stride;
    return run_attention(ctx, stream, p, k, v, seq_len - kv_start, false);
}

extern "C" int nvmai_hip_attention_decode_ragged(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                                 const nvmai_kv_view* k, const nvmai_kv_view* v,
                                                 uint64_t kv_batch_stride, void* out, uint32_t batch,
                                                 uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                                 const uint32_t* seq_lens, const uint32_t* kv_starts,
                                                 uint32_t max_seq_len, float scale) {
    AttnParams p;
    const int rc = attention_setup(ctx, q, k, v, out, batch, head_dim, num_q_heads, num_kv_heads, scale, p);
    if (rc) return rc;
    if (!seq_lens) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(q)) return NVMAI_ERR_ALIGNMENT;
    p.kv_batch_stride = kv_batch_stride;
    p.seq_len = max_seq_len; p.kv_start = 0;
    p.seq_lens = seq_lens; p.kv_starts = kv_starts;
    return run_attention(ctx, stream, p, k, v, max_seq_len, false);
}

extern "C" int nvmai_hip_attention_prefill_causal(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* q,
                                                  uint32_t q_token_stride, const nvmai_kv_view* k,
                                                  const nvmai_kv_view* v, void* out, uint32_t o_token_stride,
                                                  uint32_t start_position, uint32_t query_count,
                                                  uint32_t kv_valid_count, uint32_t sliding_window,
                                                  uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                                  uint32_t kv_ring_capacity, float scale) {
    AttnParams p;
    // PrefillAttention.validate, PrefillAttention.swift:169-191
    const int rc = attention_setup(ctx, q, k, v, out, query_count, head_dim, num_q_heads, num_kv_heads, scale, p);
    if (rc) return rc;
    if (q_token_stride < num_q_heads * head_dim || o_token_stride < num_q_heads * head_dim) return NVMAI_ERR_INVALID_ARG;
    if ((uint64_t)start_position + query_count > kv_valid_count) return NVMAI_ERR_INVALID_ARG;
    p.q_stride = q_token_stride; p.out_stride = o_token_stride;
    p.kv_batch_stride = 0;
    p.seq_len = kv_valid_count; p.kv_start = 0;
    p.causal = 1; p.causal_start = start_position; p.window = sliding_window;
    p.ring = kv_ring_capacity;
    const uint32_t longest = start_position + query_count;          // keys of the last query without a window
    const uint32_t max_len = sliding_window != 0 && sliding_window < longest ? sliding_window : longest;
    // A chunk with enough queries to give every compute unit a block of the flash-attention kernel: the key range
    // is dequantized once into fp16 scratch and that kernel runs on it (attn_prefill_kernels.hpp) -- every key
    // row is then read by hundreds of query blocks, and taking it apart once (2.6 ns per row) costs less than what
    // the kernels that multiply the codes spend per (row, query block).  Fewer queries keep those kernels, which
    // split the key range over blocks (512 queries at the end of a 32K cache: 0.64 ms against 0.98 ms on 128
    // blocks of this form); so does a range whose scratch would pass 512 MB.
    const uint32_t qpk = num_q_heads / num_kv_heads;
    const uint32_t first_a = start_position + 1u;
    const uint32_t key_lo = (sliding_window != 0u && first_a > sliding_window ? first_a - sliding_window : 0u) & ~31u;
    const uint32_t key_hi = longest < kv_valid_count ? longest : kv_valid_count;
    const uint64_t ntok = ((uint64_t)(key_hi - key_lo) + 31u) & ~(uint64_t)31u;
    const uint64_t scratch = ntok * num_kv_heads * ATTN_HD * 2;
    const bool fa_shape = head_dim == ATTN_HD && (qpk == 1 || qpk == 2 || qpk == 4 || qpk == 8 || qpk == 16);
    const uint64_t fa_blocks = fa_shape ? ((uint64_t)query_count + 64u / qpk - 1) / (64u / qpk) * num_kv_heads : 0;
    if (fa_shape && fa_blocks >= ATTN_FA_MIN_BLOCKS && scratch <= (1ull << 28) && aligned16(q) && q_token_stride % 8 == 0 && aligned16(out) &&
        o_token_stride % 8 == 0) {
        hipStream_t s = (hipStream_t)stream;
        const int wrc = ws_begin(ctx, stream, 2 * ws_round(scratch));
        if (wrc) return wrc;
        uint16_t* kd = ws_take<uint16_t>(ctx, scratch / 2);
        uint16_t* vt = ws_take<uint16_t>(ctx, scratch / 2);
        ProfScope ps(ctx, NVMAI_PROF_ATTN_PARTIAL, s);
        const AttnDequantParams dq{p.k, p.v, p.f, kv_ring_capacity, key_lo, key_hi, (uint32_t)ntok, num_kv_heads, kd, vt};
        attn_prefill_dequant_kernel<<<dim3((uint32_t)(ntok / 32), num_kv_heads), 256, 0, s>>>(dq);
        // eight waves per block (twice the queries per K / V tile fetched from the L2) when that still leaves every
        // compute unit a block, four otherwise
        const uint32_t tpw = 16u / qpk;
        const bool wide = ((uint64_t)query_count + 8u * tpw - 1) / (8u * tpw) * num_kv_heads >= ATTN_FA_MIN_BLOCKS;
        const uint32_t tpb = (wide ? 8u : 4u) * tpw;
        const dim3 grid(((query_count + tpb - 1) / tpb) * num_kv_heads);
        if (wide) {
            if (ctx->act == ACT_BF16) attn_prefill_fa_kernel<ACT_BF16, 8><<<grid, 512, 0, s>>>(p, kd, vt, (uint32_t)ntok, key_lo);
            else attn_prefill_fa_kernel<ACT_FP16, 8><<<grid, 512, 0, s>>>(p, kd, vt, (uint32_t)ntok, key_lo);
        } else {
            if (ctx->act == ACT_BF16) attn_prefill_fa_kernel<ACT_BF16, 4><<<grid, 256, 0, s>>>(p, kd, vt, (uint32_t)ntok, key_lo);
            else attn_prefill_fa_kernel<ACT_FP16, 4><<<grid, 256, 0, s>>>(p, kd, vt, (uint32_t)ntok, key_lo);
        }
        return launch_status();
    }
    return run_attention(ctx, stream, p, k, v, max_len, true);
}
