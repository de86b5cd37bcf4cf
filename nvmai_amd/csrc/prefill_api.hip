// Entry points: token-expert pairs, grouping by expert, grouped expert GEMMs, rank-order reduce.
#include "ctx.hpp"
#include "prefill_kernels.hpp"

using namespace nvmai;

static_assert(sizeof(nvmai_prefill_pair) == sizeof(PrefillPair) && sizeof(nvmai_prefill_group) == sizeof(PrefillGroup) &&
                  sizeof(nvmai_prefill_tile) == sizeof(PrefillTile),
              "C-ABI records and kernel records must agree");

extern "C" int nvmai_prefill_grouping_check(int64_t n_pairs, int64_t query_count, int64_t top_k,
                                            int64_t num_experts, int64_t tile_expert_count, int has_sort_keys,
                                            int64_t n_sort_keys) {
    if (query_count < 0) return NVMAI_GROUPING_INVALID_QUERY_COUNT;
    if (top_k <= 0) return NVMAI_GROUPING_INVALID_TOP_K;
    if (num_experts <= 0) return NVMAI_GROUPING_INVALID_NUM_EXPERTS;
    if (tile_expert_count < 1 || tile_expert_count > 16) return NVMAI_GROUPING_INVALID_TILE_EXPERT_COUNT;
    if (has_sort_keys && n_sort_keys != num_experts) return NVMAI_GROUPING_SORT_KEY_COUNT_MISMATCH;
    if (n_pairs != query_count * top_k) return NVMAI_GROUPING_PAIR_COUNT_MISMATCH;
    return NVMAI_GROUPING_OK;
}

extern "C" int nvmai_hip_prefill_make_pairs(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint32_t* idx,
                                            const uint16_t* w, uint32_t tokens, uint32_t top_k,
                                            nvmai_prefill_pair* pairs) {
    if (!ctx || !idx || !w || !pairs || top_k == 0) return NVMAI_ERR_INVALID_ARG;
    const uint64_t n = (uint64_t)tokens * top_k;
    if (n >= (1u << 28)) return NVMAI_ERR_INVALID_ARG;
    if (n == 0) return NVMAI_OK;
    prefill_make_pairs_kernel<<<(uint32_t)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        idx, w, (uint32_t)n, top_k, reinterpret_cast<PrefillPair*>(pairs));
    return launch_status();
}

namespace {

constexpr uint32_t MAX_GROUP_EXPERTS = 2048;   // five u32 arrays of the scan kernel in 40 KB of LDS
constexpr int ERR_WORD = 8;                    // index into the context's persistent zeroed words

int check_grouping(const nvmai_prefill_grouping* g, uint64_t n_pairs) {
    if (!g || (n_pairs && !g->sorted_pairs) || !g->expert_offsets || !g->expert_counts || !g->groups || !g->tiles || !g->info)
        return NVMAI_ERR_INVALID_ARG;
    return NVMAI_OK;
}

// Shared tail: histogram, scan, scatter over slot-ordered expert ids.
int group_slots(nvmai_hip_ctx* ctx, hipStream_t s, const uint32_t* slot_expert, const uint32_t* w32,
                const uint16_t* w16, uint32_t n_pairs, uint32_t top_k, uint32_t num_experts,
                uint32_t tile_expert_count, const uint64_t* sort_keys, uint32_t* block_hist, uint32_t* block_base,
                uint32_t* words, bool report_range, const nvmai_prefill_grouping* out) {
    const uint32_t n_blocks = (n_pairs + GROUP_CHUNK - 1) / GROUP_CHUNK;
    if (n_blocks)
        prefill_hist_kernel<<<n_blocks, 256, num_experts * 4, s>>>(slot_expert, n_pairs, num_experts, block_hist, words,
                                                                  report_range);
    if (n_blocks && n_blocks <= FUSED_MAX_BLOCKS && num_experts <= FUSED_MAX_EXPERTS) {
        uint32_t id_bits = 0;
        while ((1u << id_bits) < num_experts) ++id_bits;
        prefill_scan_scatter_kernel<<<n_blocks, 256, (12 * num_experts + 8) * 4, s>>>(
            slot_expert, w32, w16, n_pairs, top_k, num_experts, id_bits, block_hist, n_blocks, sort_keys, tile_expert_count,
            out->expert_offsets, out->expert_counts, reinterpret_cast<PrefillGroup*>(out->groups),
            reinterpret_cast<PrefillTile*>(out->tiles), words, out->info, reinterpret_cast<PrefillPair*>(out->sorted_pairs));
        return launch_status();
    }
    prefill_scan_kernel<<<1, 1024, (5 * num_experts + 32) * 4, s>>>(
        block_hist, block_base, n_blocks, num_experts, sort_keys, tile_expert_count, out->expert_offsets, out->expert_counts,
        reinterpret_cast<PrefillGroup*>(out->groups), reinterpret_cast<PrefillTile*>(out->tiles), words, out->info);
    if (n_blocks)
        prefill_scatter_kernel<<<n_blocks, 256, num_experts * 4, s>>>(slot_expert, w32, w16, n_pairs, top_k, num_experts,
                                                                    block_base, reinterpret_cast<PrefillPair*>(out->sorted_pairs));
    return launch_status();
}

}  // namespace

extern "C" int nvmai_hip_prefill_group_pairs(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                             const nvmai_prefill_pair* pairs, uint64_t n_pairs,
                                             uint32_t query_count, uint32_t top_k, uint32_t num_experts,
                                             uint32_t tile_expert_count, const uint64_t* sort_keys,
                                             uint64_t n_sort_keys, const nvmai_prefill_grouping* out) {
    if (!ctx || (n_pairs && !pairs)) return NVMAI_ERR_INVALID_ARG;
    int rc = check_grouping(out, n_pairs);
    if (rc) return rc;
    if (nvmai_prefill_grouping_check((int64_t)n_pairs, query_count, top_k, num_experts, tile_expert_count,
                                     sort_keys != nullptr, (int64_t)n_sort_keys) != NVMAI_GROUPING_OK)
        return NVMAI_ERR_INVALID_ARG;
    if (n_pairs >= (1u << 28) || num_experts > MAX_GROUP_EXPERTS) return NVMAI_ERR_UNSUPPORTED;
    const uint32_t n = (uint32_t)n_pairs, n_blocks = (n + GROUP_CHUNK - 1) / GROUP_CHUNK;
    rc = ws_begin(ctx, stream, 3 * ws_round((size_t)n * 4) + 2 * ws_round((size_t)n_blocks * num_experts * 4));
    if (rc) return rc;
    uint32_t* first = ws_take<uint32_t>(ctx, n);
    uint32_t* slot_expert = ws_take<uint32_t>(ctx, n);
    uint32_t* slot_weight = ws_take<uint32_t>(ctx, n);
    uint32_t* block_hist = ws_take<uint32_t>(ctx, (size_t)n_blocks * num_experts);
    uint32_t* block_base = ws_take<uint32_t>(ctx, (size_t)n_blocks * num_experts);
    uint32_t* words = ctx->tickets + ERR_WORD;
    hipStream_t s = (hipStream_t)stream;
    ProfScope prof(ctx, NVMAI_PROF_PREFILL_GROUP, s);
    const uint32_t grid = (n + 255) / 256;
    if (n) {
        prefill_init_kernel<<<grid, 256, 0, s>>>(first, n);
        prefill_claim_kernel<<<grid, 256, 0, s>>>(reinterpret_cast<const PrefillPair*>(pairs), n, query_count, top_k,
                                                  num_experts, first, words);
        prefill_slot_kernel<<<grid, 256, 0, s>>>(reinterpret_cast<const PrefillPair*>(pairs), n, query_count, top_k,
                                                 num_experts, first, slot_expert, slot_weight, words);
    }
    return group_slots(ctx, s, slot_expert, slot_weight, nullptr, n, top_k, num_experts, tile_expert_count, sort_keys,
                       block_hist, block_base, words, false, out);
}

extern "C" int nvmai_hip_prefill_group_routes(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint32_t* idx,
                                              const uint16_t* w, uint32_t query_count, uint32_t top_k,
                                              uint32_t num_experts, uint32_t tile_expert_count,
                                              const uint64_t* sort_keys, uint64_t n_sort_keys,
                                              const nvmai_prefill_grouping* out) {
    const uint64_t n_pairs = (uint64_t)query_count * top_k;
    if (!ctx || (n_pairs && (!idx || !w))) return NVMAI_ERR_INVALID_ARG;
    int rc = check_grouping(out, n_pairs);
    if (rc) return rc;
    if (nvmai_prefill_grouping_check((int64_t)n_pairs, query_count, top_k, num_experts, tile_expert_count,
                                     sort_keys != nullptr, (int64_t)n_sort_keys) != NVMAI_GROUPING_OK)
        return NVMAI_ERR_INVALID_ARG;
    if (n_pairs >= (1u << 28) || num_experts > MAX_GROUP_EXPERTS) return NVMAI_ERR_UNSUPPORTED;
    const uint32_t n = (uint32_t)n_pairs, n_blocks = (n + GROUP_CHUNK - 1) / GROUP_CHUNK;
    rc = ws_begin(ctx, stream, 2 * ws_round((size_t)n_blocks * num_experts * 4));
    if (rc) return rc;
    uint32_t* block_hist = ws_take<uint32_t>(ctx, (size_t)n_blocks * num_experts);
    uint32_t* block_base = ws_take<uint32_t>(ctx, (size_t)n_blocks * num_experts);
    hipStream_t s = (hipStream_t)stream;
    ProfScope prof(ctx, NVMAI_PROF_PREFILL_GROUP, s);
    return group_slots(ctx, s, idx, nullptr, w, n, top_k, num_experts, tile_expert_count, sort_keys, block_hist,
                       block_base, ctx->tickets + ERR_WORD, true, out);
}

namespace {

// Blocks of a dense launch over `tiles` M tiles: eight XCDs times the most any of them owns (M tiles dealt over
// the XCDs from eight tiles on, column tiles otherwise; prefill_gemm_kernel).
uint32_t gemm_grid(uint32_t tiles, const GemmParams& g) {
    const uint32_t per_xcd = tiles >= 8 ? (tiles + 7) / 8 * g.n_tiles_n : (g.n_tiles_n + 7) / 8 * tiles;
    return GEMM_XCDS * per_xcd;
}

// Blocks of a grouped launch.  The work lists are dealt in serpentine order from a sorted sequence of
// items of at most max(2, ceil(tiles / 64)) M tiles, so no list is longer than an eighth of the
// tiles plus one item; every column tile of every list position is a block, and blocks past the
// end of their list leave at once.
uint32_t grouped_list_max(uint32_t max_mtiles) { return (max_mtiles + 7) / 8 + (max_mtiles + 63) / 64 + 2; }
uint32_t grouped_grid(uint32_t max_mtiles, const GemmParams& g) {
    return GEMM_XCDS * grouped_list_max(max_mtiles) * g.n_tiles_n;
}

// Rows per M tile of a dense product.  A launch of at most 128 blocks of 128 rows leaves half of the compute
// units idle; tiles of 64 rows (the same kernel's four-row-tile body) double the blocks: the shared expert's
// gate/up product over 4096 rows 46 -> 38 us.  At 256 blocks -- one per unit where two fit -- the shorter
// tiles were measured too and do not pay (2048 x 4096 over 4096 rows: 98 -> 107 us; 2048 x 512: 22 us both ways).
uint32_t dense_bm_for(uint32_t rows, uint32_t n_tiles_n) {
    const uint64_t blocks = (uint64_t)((rows + GEMM_BM - 1) / GEMM_BM) * n_tiles_n;
    return rows > 64 && blocks <= 128 ? 64u : (uint32_t)GEMM_BM;
}
uint32_t dense_tiles(const GemmParams& g) { return (g.dense_rows + g.dense_bm - 1) / g.dense_bm; }

// dense: grid over the M tiles the kernel cuts itself; grouped: a block per column tile of every list position
// of at most `tiles` M tiles.
template <int ACT, int BITS, int NT>
void launch_gemms(const GemmParams& g1, const GemmParams& g2, uint32_t tiles, nvmai_hip_ctx* ctx, hipStream_t s) {
    const bool dense = g1.dense_rows != 0;
    {
        ProfScope prof(ctx, NVMAI_PROF_PREFILL_GEMM1, s);
        prefill_gemm_kernel<ACT, BITS, true, NT><<<dense ? gemm_grid(dense_tiles(g1), g1) : grouped_grid(tiles, g1), 256, 0, s>>>(g1);
    }
    {
        ProfScope prof(ctx, NVMAI_PROF_PREFILL_GEMM2, s);
        prefill_gemm_kernel<ACT, BITS, false, NT><<<dense ? gemm_grid(dense_tiles(g2), g2) : grouped_grid(tiles, g2), 256, 0, s>>>(g2);
    }
}

}  // namespace

// One expert over every row of x (the shared expert of a prefill block): gate/up + SwiGLU and
// down through the grouped-GEMM kernels in their dense mode, then the optional scalar gate.
// x [tokens, x_stride] and y [tokens, y_stride] in the context's activation type; act and tmp
// are 16-bit scratch [tokens, f] and [tokens, d], 16-byte aligned.
namespace nvmai {
int expert_ffn_dense(nvmai_hip_ctx* ctx, hipStream_t s, const uint8_t* blob, const nvmai_expert_offsets* off,
                     uint32_t bits, const void* x, uint32_t x_stride, uint32_t tokens, uint32_t d, uint32_t f,
                     void* act, void* tmp, const float* gate_logit, void* y, uint32_t y_stride) {
    const uint32_t nt = bits == 4 ? 4 : 2;
    const uint32_t tiles = (tokens + GEMM_BM - 1) / GEMM_BM;
    GemmParams g1{};
    g1.pool = blob; g1.pool_stride = 0x7FFFFFFFull;   // bound of the scale resources; the only "expert" is 0
    g1.wA = off->gate_w; g1.sA = off->gate_s; g1.bA = off->gate_b;
    g1.wB = off->up_w; g1.sB = off->up_s; g1.bB = off->up_b;
    g1.dense_rows = tokens;
    g1.x = x; g1.x_stride = x_stride; g1.out = act; g1.out_stride = f;
    g1.K = d; g1.N = f; g1.top_k = 1; g1.n_tiles_n = (f + 32 * nt - 1) / (32 * nt);
    g1.dense_bm = dense_bm_for(tokens, g1.n_tiles_n);
    GemmParams g2 = g1;
    g2.wA = off->down_w; g2.sA = off->down_s; g2.bA = off->down_b;
    g2.wB = g2.sB = g2.bB = 0;
    g2.x = act; g2.x_stride = f; g2.out = tmp; g2.out_stride = d;
    g2.K = f; g2.N = d; g2.n_tiles_n = (d + 64 * nt - 1) / (64 * nt);
    g2.dense_bm = dense_bm_for(tokens, g2.n_tiles_n);
    if (ctx->act == ACT_BF16) {
        if (bits == 4) launch_gemms<ACT_BF16, 4, 4>(g1, g2, tiles, ctx, s);
        else launch_gemms<ACT_BF16, 8, 2>(g1, g2, tiles, ctx, s);
    } else {
        if (bits == 4) launch_gemms<ACT_FP16, 4, 4>(g1, g2, tiles, ctx, s);
        else launch_gemms<ACT_FP16, 8, 2>(g1, g2, tiles, ctx, s);
    }
    if (d % 8 == 0 && y_stride % 8 == 0 && aligned16(tmp) && aligned16(y)) {       // sixteen bytes per thread
        dim3 grid8((d / 8 + 255) / 256, tokens);
        if (ctx->act == ACT_BF16)
            gate_rows8_kernel<ACT_BF16><<<grid8, 256, 0, s>>>((const uint16_t*)tmp, gate_logit, (uint16_t*)y, tokens, d, y_stride);
        else
            gate_rows8_kernel<ACT_FP16><<<grid8, 256, 0, s>>>((const uint16_t*)tmp, gate_logit, (uint16_t*)y, tokens, d, y_stride);
        return launch_status();
    }
    dim3 grid((d + 255) / 256, tokens);
    if (ctx->act == ACT_BF16)
        gate_rows_kernel<ACT_BF16><<<grid, 256, 0, s>>>((const uint16_t*)tmp, gate_logit, (uint16_t*)y, tokens, d, y_stride);
    else
        gate_rows_kernel<ACT_FP16><<<grid, 256, 0, s>>>((const uint16_t*)tmp, gate_logit, (uint16_t*)y, tokens, d, y_stride);
    return launch_status();
}
}  // namespace nvmai

extern "C" int nvmai_hip_prefill_grouped_moe(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* experts_base,
                                             uint64_t expert_stride, const nvmai_expert_offsets* off,
                                             uint32_t bits, uint32_t d, uint32_t f, uint32_t num_experts,
                                             const void* hidden, uint32_t hidden_stride, uint32_t query_count,
                                             uint32_t top_k, const nvmai_prefill_grouping* grouping,
                                             void* act_scratch, void* route_partials) {
    if (!ctx || !experts_base || !off || !hidden || !act_scratch || !route_partials) return NVMAI_ERR_INVALID_ARG;
    int rc = check_grouping(grouping, (uint64_t)query_count * top_k);
    if (rc) return rc;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (d == 0 || f == 0 || d % NVMAI_GROUP || f % NVMAI_GROUP || top_k == 0 || num_experts == 0 ||
        hidden_stride < d)
        return NVMAI_ERR_INVALID_ARG;
    const uint32_t offs[9] = {off->gate_w, off->gate_s, off->gate_b, off->up_w, off->up_s, off->up_b,
                              off->down_w, off->down_s, off->down_b};
    for (int i = 0; i < 9; ++i)
        if (offs[i] % (i % 3 == 0 ? 16 : 2)) return NVMAI_ERR_ALIGNMENT;
    if (!aligned16(experts_base) || expert_stride % 16 || !aligned16(hidden) || hidden_stride % 8 ||
        !aligned16(act_scratch) || !aligned16(route_partials))
        return NVMAI_ERR_ALIGNMENT;
    const uint64_t n_pairs = (uint64_t)query_count * top_k;
    if (n_pairs >= (1u << 28)) return NVMAI_ERR_UNSUPPORTED;
    // the GEMM kernel addresses every operand array with 32-bit byte offsets
    if ((uint64_t)query_count * hidden_stride * 2 > 0xFFFFFFFFull || n_pairs * f * 2 > 0xFFFFFFFFull ||
        (uint64_t)d * f * bits / 8 > 0xFFFFFFFFull)
        return NVMAI_ERR_UNSUPPORTED;
    if (n_pairs == 0) return NVMAI_OK;
    // full tiles + one remainder per expert: what all eight work lists hold together, and a bound
    // for each of them
    const uint32_t max_mtiles = (uint32_t)(n_pairs / GEMM_BM) + (num_experts < n_pairs ? num_experts : (uint32_t)n_pairs);
    rc = ws_begin(ctx, stream, ws_round((size_t)GEMM_XCDS * max_mtiles * sizeof(MTile)) + ws_round(GEMM_XCDS * 4));
    if (rc) return rc;
    MTile* mtiles = ws_take<MTile>(ctx, (size_t)GEMM_XCDS * max_mtiles);
    uint32_t* qwords = ws_take<uint32_t>(ctx, GEMM_XCDS);   // list lengths
    hipStream_t s = (hipStream_t)stream;
    prefill_mtiles_kernel<<<1, 256, 0, s>>>(reinterpret_cast<const PrefillGroup*>(grouping->groups), grouping->info,
                                            mtiles, max_mtiles, grouped_list_max(max_mtiles), qwords,
                                            reinterpret_cast<uint4*>(route_partials),
                                            n_pairs * d * 2 / 16);
    const uint32_t nt = bits == 4 ? 4 : 2;        // 16-column tiles per wave: what the register file allows
    GemmParams g1{};
    g1.pool = (const uint8_t*)experts_base; g1.pool_stride = expert_stride;
    g1.wA = off->gate_w; g1.sA = off->gate_s; g1.bA = off->gate_b;
    g1.wB = off->up_w; g1.sB = off->up_s; g1.bB = off->up_b;
    g1.mtiles = mtiles; g1.list_cap = max_mtiles; g1.list_len = qwords;
    g1.pairs = reinterpret_cast<const PrefillPair*>(grouping->sorted_pairs);
    g1.x = hidden; g1.x_stride = hidden_stride;
    g1.out = act_scratch; g1.out_stride = f;
    g1.K = d; g1.N = f; g1.top_k = top_k; g1.n_tiles_n = (f + 32 * nt - 1) / (32 * nt);
    GemmParams g2 = g1;
    g2.wA = off->down_w; g2.sA = off->down_s; g2.bA = off->down_b;
    g2.wB = g2.sB = g2.bB = 0;
    g2.x = act_scratch; g2.x_stride = f;
    g2.out = route_partials; g2.out_stride = d;
    g2.K = f; g2.N = d; g2.n_tiles_n = (d + 64 * nt - 1) / (64 * nt);
    if (ctx->act == ACT_BF16) {
        if (bits == 4) launch_gemms<ACT_BF16, 4, 4>(g1, g2, max_mtiles, ctx, s);
        else launch_gemms<ACT_BF16, 8, 2>(g1, g2, max_mtiles, ctx, s);
    } else {
        if (bits == 4) launch_gemms<ACT_FP16, 4, 4>(g1, g2, max_mtiles, ctx, s);
        else launch_gemms<ACT_FP16, 8, 2>(g1, g2, max_mtiles, ctx, s);
    }
    return launch_status();
}

// One streamed tile: PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:413-489)
// with the tile's experts bound through separate blobs.
extern "C" int nvmai_hip_prefill_grouped_moe_streamed(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                                      const nvmai_prefill_streamed_params* params,
                                                      const void* const* expert_blobs, uint32_t bits,
                                                      const void* hidden, const nvmai_prefill_pair* sorted_pairs,
                                                      uint64_t n_sorted_pairs, void* act_scratch, void* route_partials,
                                                      uint32_t* err) {
    static_assert(sizeof(nvmai_prefill_streamed_params) == 128, "PrefillGroupedRoutedMoEStreamedParams is 128 bytes");
    if (!ctx || !params || !expert_blobs || !hidden || !sorted_pairs || !act_scratch || !route_partials)
        return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    const uint32_t d = params->d, f = params->routed_intermediate, top_k = params->top_k;
    const uint32_t live = params->live_expert_count;
    // PrefillStreamedTileBinding.init (PrefillGroupedRoutedMoE.swift:189-214): 1 .. 16 experts, ids unique
    if (live == 0 || live > STREAMED_MAX_EXPERTS) return NVMAI_ERR_INVALID_ARG;
    for (uint32_t i = 0; i < live; ++i) {
        if (!expert_blobs[i] || params->local_expert[i] == 0xFFFFFFFFu) return NVMAI_ERR_INVALID_ARG;
        if (!aligned16(expert_blobs[i])) return NVMAI_ERR_ALIGNMENT;
        for (uint32_t j = 0; j < i; ++j)
            if (params->local_expert[j] == params->local_expert[i]) return NVMAI_ERR_INVALID_ARG;
    }
    if (d == 0 || f == 0 || d % NVMAI_GROUP || f % NVMAI_GROUP || top_k == 0 || params->hidden_stride_elements < d)
        return NVMAI_ERR_INVALID_ARG;
    // validateCoversPairs' range check (:274-279)
    if ((uint64_t)params->pair_start + params->pair_count > n_sorted_pairs) return NVMAI_ERR_INVALID_ARG;
    const uint32_t offs[9] = {params->gate_w_off, params->gate_s_off, params->gate_b_off, params->up_w_off,
                              params->up_s_off, params->up_b_off, params->down_w_off, params->down_s_off,
                              params->down_b_off};
    for (int i = 0; i < 9; ++i)
        if (offs[i] % (i % 3 == 0 ? 16 : 2)) return NVMAI_ERR_ALIGNMENT;
    if (!aligned16(hidden) || params->hidden_stride_elements % 8 || !aligned16(act_scratch) || !aligned16(route_partials))
        return NVMAI_ERR_ALIGNMENT;
    if (n_sorted_pairs >= (1u << 28)) return NVMAI_ERR_UNSUPPORTED;
    if (n_sorted_pairs * f * 2 > 0xFFFFFFFFull || n_sorted_pairs * d * 2 > 0xFFFFFFFFull ||
        (uint64_t)d * f * bits / 8 > 0xFFFFFFFFull)
        return NVMAI_ERR_UNSUPPORTED;
    if (params->pair_count == 0) return NVMAI_OK;
    // the extent of a blob, from its last array: the bound of the kernel's scale / bias resources
    uint64_t extent = 0;
    const uint64_t w_bytes = (uint64_t)d * f * bits / 8, gu_meta = (uint64_t)f * (d / NVMAI_GROUP) * 2,
                   dn_meta = (uint64_t)d * (f / NVMAI_GROUP) * 2;
    const uint64_t ends[9] = {offs[0] + w_bytes, offs[1] + gu_meta, offs[2] + gu_meta, offs[3] + w_bytes, offs[4] + gu_meta,
                              offs[5] + gu_meta, offs[6] + w_bytes, offs[7] + dn_meta, offs[8] + dn_meta};
    for (int i = 0; i < 9; ++i) extent = ends[i] > extent ? ends[i] : extent;
    if (extent > 0xFFFFFFFFull) return NVMAI_ERR_UNSUPPORTED;
    const uint32_t max_mtiles = params->pair_count / GEMM_BM + live;
    int rc = ws_begin(ctx, stream, ws_round((size_t)GEMM_XCDS * max_mtiles * sizeof(MTile)) + ws_round(GEMM_XCDS * 4) +
                                       ws_round(STREAMED_MAX_EXPERTS * sizeof(void*)));
    if (rc) return rc;
    MTile* mtiles = ws_take<MTile>(ctx, (size_t)GEMM_XCDS * max_mtiles);
    uint32_t* qwords = ws_take<uint32_t>(ctx, GEMM_XCDS);
    const uint8_t** table = ws_take<const uint8_t*>(ctx, STREAMED_MAX_EXPERTS);
    StreamedBind b{};
    for (uint32_t i = 0; i < live; ++i) { b.blob[i] = (const uint8_t*)expert_blobs[i]; b.expert[i] = params->local_expert[i]; }
    b.live = live; b.pair_start = params->pair_start; b.pair_count = params->pair_count;
    hipStream_t s = (hipStream_t)stream;
    prefill_streamed_mtiles_kernel<<<1, 256, 0, s>>>(reinterpret_cast<const PrefillPair*>(sorted_pairs), b, table, mtiles,
                                                     max_mtiles, qwords, err);
    const uint32_t nt = bits == 4 ? 4 : 2;
    GemmParams g1{};
    g1.pool = nullptr; g1.pool_stride = extent; g1.blob_table = table;
    g1.wA = offs[0]; g1.sA = offs[1]; g1.bA = offs[2];
    g1.wB = offs[3]; g1.sB = offs[4]; g1.bB = offs[5];
    g1.mtiles = mtiles; g1.list_cap = max_mtiles; g1.list_len = qwords;
    g1.pairs = reinterpret_cast<const PrefillPair*>(sorted_pairs);
    g1.x = hidden; g1.x_stride = params->hidden_stride_elements;
    g1.out = act_scratch; g1.out_stride = f;
    g1.K = d; g1.N = f; g1.top_k = top_k; g1.n_tiles_n = (f + 32 * nt - 1) / (32 * nt);
    GemmParams g2 = g1;
    g2.wA = offs[6]; g2.sA = offs[7]; g2.bA = offs[8];
    g2.wB = g2.sB = g2.bB = 0;
    g2.x = act_scratch; g2.x_stride = f;
    g2.out = route_partials; g2.out_stride = d;
    g2.K = f; g2.N = d; g2.n_tiles_n = (d + 64 * nt - 1) / (64 * nt);
    if (ctx->act == ACT_BF16) {
        if (bits == 4) launch_gemms<ACT_BF16, 4, 4>(g1, g2, max_mtiles, ctx, s);
        else launch_gemms<ACT_BF16, 8, 2>(g1, g2, max_mtiles, ctx, s);
    } else {
        if (bits == 4) launch_gemms<ACT_FP16, 4, 4>(g1, g2, max_mtiles, ctx, s);
        else launch_gemms<ACT_FP16, 8, 2>(g1, g2, max_mtiles, ctx, s);
    }
    return launch_status();
}

namespace {
template <int ACT, int BITS, int NT>
void launch_qmm(const GemmParams& g, uint32_t blocks, hipStream_t s) {
    prefill_gemm_kernel<ACT, BITS, false, NT><<<blocks, 256, 0, s>>>(g);
}
}  // namespace

extern "C" int nvmai_hip_affine_qmm(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint8_t* weights,
                                    const uint16_t* scales, const uint16_t* biases, uint32_t bits,
                                    const void* x, uint32_t x_stride, void* y, uint32_t y_stride, uint32_t m,
                                    uint32_t n, uint32_t k) {
    if (!ctx || !weights || !scales || !biases || !x || !y) return NVMAI_ERR_INVALID_ARG;
    if (bits != 4 && bits != 8) return NVMAI_ERR_UNSUPPORTED;
    if (n == 0 || k == 0 || k % NVMAI_GROUP || x_stride < k || y_stride < n) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(weights) || !aligned16(x) || x_stride % 8 || !aligned16(y) ||
        (reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 1u)
        return NVMAI_ERR_ALIGNMENT;
    if (m == 0) return NVMAI_OK;
    if (m >= (1u << 28)) return NVMAI_ERR_UNSUPPORTED;
    // the GEMM kernel addresses every operand array with 32-bit byte offsets
    if ((uint64_t)m * x_stride * 2 > 0xFFFFFFFFull || (uint64_t)n * k * bits / 8 > 0xFFFFFFFFull)
        return NVMAI_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    ProfScope prof(ctx, NVMAI_PROF_PREFILL_GEMM2, s);
    const uint32_t nt = bits == 4 ? 4 : 2;
    GemmParams g{};
    g.pool = weights; g.pool_stride = 0;
    g.wA = 0;
    g.sA = reinterpret_cast<const uint8_t*>(scales) - weights;
    g.bA = reinterpret_cast<const uint8_t*>(biases) - weights;
    g.dense_rows = m;                           // the kernel cuts the rows into M tiles itself
    g.x = x; g.x_stride = x_stride; g.out = y; g.out_stride = y_stride;
    g.K = k; g.N = n; g.top_k = 1; g.n_tiles_n = (n + 64 * nt - 1) / (64 * nt);
    g.dense_bm = dense_bm_for(m, g.n_tiles_n);
    const uint32_t blocks = gemm_grid(dense_tiles(g), g);
    if (ctx->act == ACT_BF16) { if (bits == 4) launch_qmm<ACT_BF16, 4, 4>(g, blocks, s); else launch_qmm<ACT_BF16, 8, 2>(g, blocks, s); }
    else { if (bits == 4) launch_qmm<ACT_FP16, 4, 4>(g, blocks, s); else launch_qmm<ACT_FP16, 8, 2>(g, blocks, s); }
    return launch_status();
}

extern "C" int nvmai_hip_prefill_moe_reduce_token_major(nvmai_hip_ctx* ctx, nvmai_stream stream,
                                                        const void* route_partials, const uint16_t* route_weights,
                                                        void* h2, uint32_t h2_stride, uint32_t query_count,
                                                        uint32_t top_k, uint32_t d) {
    if (!ctx || !route_partials || !route_weights || !h2) return NVMAI_ERR_INVALID_ARG;
    if (query_count == 0 || top_k == 0 || d == 0 || d % 2 || h2_stride < d || h2_stride % 2) return NVMAI_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    ProfScope prof(ctx, NVMAI_PROF_PREFILL_COMBINE, s);
    const bool vec = d % 8 == 0 && h2_stride % 8 == 0 && aligned16(route_partials) && aligned16(h2);
    const uint32_t per = vec ? 8 : 2;
    dim3 grid((d / per + 255) / 256, query_count);
#define NVMAI_REDUCE(ACT, VEC) \
    prefill_reduce_kernel<ACT, VEC><<<grid, 256, 0, s>>>(route_partials, route_weights, h2, query_count, top_k, d, h2_stride)
    if (ctx->act == ACT_BF16) { if (vec) NVMAI_REDUCE(ACT_BF16, 8); else NVMAI_REDUCE(ACT_BF16, 2); }
    else { if (vec) NVMAI_REDUCE(ACT_FP16, 8); else NVMAI_REDUCE(ACT_FP16, 2); }
#undef NVMAI_REDUCE
    return launch_status();
}
