// Entry points: tiled softmax over the vocabulary, top-64 and generic samplers.
#include <time.h>

#include <atomic>

#include "ctx.hpp"
#include "sample_kernels.hpp"

using namespace nvmai;

// first of SAMPLE_MAX_ROWS persistent zeroed words of the context used as per-row block counters
constexpr int GUMBEL_TICKETS = 16;

extern "C" uint64_t nvmai_sampler_seed_for(uint64_t seed, int64_t position) {
    uint64_t z = seed + (uint64_t)position + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return z == 0 ? 0x9E3779B97F4A7C15ull : z;
}

extern "C" int nvmai_hip_softmax_tiled(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* logits,
                                       uint32_t logits_stride, uint16_t* probs, uint32_t probs_stride,
                                       uint32_t rows, uint32_t v, float softcap) {
    if (!ctx || !logits || !probs || v == 0 || logits_stride < v || probs_stride < v) return NVMAI_ERR_INVALID_ARG;
    if (rows == 0) return NVMAI_OK;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t tiles = (v + SOFTMAX_TILE - 1) / SOFTMAX_TILE;
    int rc = ws_begin(ctx, stream, 2 * ws_round((size_t)rows * tiles * 4));
    if (rc) return rc;
    float* tmax = ws_take<float>(ctx, (size_t)rows * tiles);
    float* tsum = ws_take<float>(ctx, (size_t)rows * tiles);
    ProfScope ps(ctx, NVMAI_PROF_SOFTMAX, s);
    dim3 grid(tiles, rows);
    if (ctx->act == ACT_BF16) {
        softmax_stage1_kernel<ACT_BF16><<<grid, 256, 0, s>>>(logits, v, logits_stride, softcap, tmax, tsum, tiles);
        softmax_normalize_kernel<ACT_BF16><<<grid, 256, 0, s>>>(logits, v, logits_stride, softcap, tmax, tsum, tiles, probs, probs_stride);
    } else {
        softmax_stage1_kernel<ACT_FP16><<<grid, 256, 0, s>>>(logits, v, logits_stride, softcap, tmax, tsum, tiles);
        softmax_normalize_kernel<ACT_FP16><<<grid, 256, 0, s>>>(logits, v, logits_stride, softcap, tmax, tsum, tiles, probs, probs_stride);
    }
    return launch_status();
}

extern "C" int nvmai_hip_sample_topk64(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint16_t* probs,
                                       uint32_t probs_stride, uint32_t rows, uint32_t v, float temperature,
                                       float top_p, const uint64_t* seeds, uint32_t top_k, uint32_t* out_token,
                                       uint32_t* top64_out) {
    if (!ctx || !probs || !seeds || !out_token || probs_stride < v) return NVMAI_ERR_INVALID_ARG;
    if (v == 0 || v > 262144) return NVMAI_ERR_UNSUPPORTED;      // SampleTopK64Error.unsupportedVocabulary
    if (!(temperature > 0.0f)) return NVMAI_ERR_INVALID_ARG;     // LogitOutput.swift:280-281
    if (top_k < 1 || top_k > 64) return NVMAI_ERR_INVALID_ARG;   // LogitOutput.swift:282-283
    if (rows == 0) return NVMAI_OK;
    if (rows > SAMPLE_MAX_ROWS) return NVMAI_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t g1 = (v + SAMPLE_TILE - 1) / SAMPLE_TILE, c1 = g1 * SAMPLE_KEEP;
    const uint32_t g2 = (c1 + SAMPLE_TILE - 1) / SAMPLE_TILE, c2 = g2 * SAMPLE_KEEP;
    int rc = ws_begin(ctx, stream, ws_round((size_t)rows * c1 * 8) + ws_round((size_t)rows * c2 * 8));
    if (rc) return rc;
    uint64_t* s1 = ws_take<uint64_t>(ctx, (size_t)rows * c1);
    uint64_t* s2 = ws_take<uint64_t>(ctx, (size_t)rows * c2);
    SeedArray sa{};
    for (uint32_t r = 0; r < rows; ++r) sa.s[r] = seeds[r];
    ProfScope ps(ctx, NVMAI_PROF_SAMPLE, s);
    sample_topk64_stage1_kernel<<<dim3(g1, rows), 256, 0, s>>>(probs, v, probs_stride, s1, c1);
    sample_topk64_reduce_kernel<<<dim3(g2, rows), 256, 0, s>>>(s1, c1, c1, s2, c2);
    sample_topk64_final_kernel<<<dim3(rows), 256, 0, s>>>(s2, c2, c2, temperature, top_p, sa, top_k, out_token, top64_out);
    return launch_status();
}

extern "C" int nvmai_hip_sample(nvmai_hip_ctx* ctx, nvmai_stream stream, const uint16_t* probs,
                                uint32_t probs_stride, uint32_t rows, uint32_t v, float temperature,
                                uint32_t top_k, float top_p, const uint64_t* seeds, const uint32_t* positions,
                                uint32_t* out_token) {
    if (!ctx || !probs || !seeds || !out_token || v == 0 || probs_stride < v) return NVMAI_ERR_INVALID_ARG;
    if (rows == 0) return NVMAI_OK;
    if (rows > SAMPLE_MAX_ROWS) return NVMAI_ERR_INVALID_ARG;
    SeedArray sa{};
    for (uint32_t r = 0; r < rows; ++r) sa.s[r] = seeds[r];
    hipStream_t s = (hipStream_t)stream;
    ProfScope ps(ctx, NVMAI_PROF_SAMPLE, s);
    if (temperature > 0.0f && top_k == 0u && (top_p <= 0.0f || top_p >= 1.0f)) {   // logit.metal:391
        PosArray pa{};
        for (uint32_t r = 0; r < rows; ++r) pa.p[r] = positions ? positions[r] : 0u;
        const int rc = ws_begin(ctx, stream, ws_round((size_t)rows * GUMBEL_BLOCKS * 8));
        if (rc) return rc;
        uint64_t* block_best = ws_take<uint64_t>(ctx, (size_t)rows * GUMBEL_BLOCKS);
        sample_gumbel_kernel<<<dim3(GUMBEL_BLOCKS, rows), 256, 0, s>>>(probs, v, probs_stride, temperature, sa, pa,
                                                                      block_best, ctx->tickets + GUMBEL_TICKETS,
                                                                      out_token);
        return launch_status();
    }
    sample_generic_kernel<<<dim3(rows), 256, 0, s>>>(probs, v, probs_stride, temperature, top_k, top_p, sa, out_token);
    return launch_status();
}

extern "C" int nvmai_hip_repetition_penalty(nvmai_hip_ctx* ctx, nvmai_stream stream, void* logits, uint32_t v,
                                            const int32_t* history_ids, uint32_t n_ids, float penalty,
                                            float logit_softcap) {
    if (!ctx || !logits || v == 0 || (n_ids && !history_ids)) return NVMAI_ERR_INVALID_ARG;
    if (!(penalty > 0.0f)) return NVMAI_ERR_INVALID_ARG;
    if (n_ids == 0 || penalty == 1.0f) return NVMAI_OK;          // Sampler.swift:181
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((n_ids + 255) / 256);
    const int rc = ws_begin(ctx, stream, ws_round((size_t)n_ids * 2));     // the snapshot: two bytes per history entry
    if (rc) return rc;
    uint16_t* snapshot = ws_take<uint16_t>(ctx, n_ids);
    repetition_penalty_gather_kernel<<<grid, 256, 0, s>>>((const uint16_t*)logits, v, history_ids, n_ids, snapshot);
    if (ctx->act == ACT_BF16)
        repetition_penalty_kernel<ACT_BF16><<<grid, 256, 0, s>>>((uint16_t*)logits, v, history_ids, n_ids, snapshot, penalty, logit_softcap);
    else
        repetition_penalty_kernel<ACT_FP16><<<grid, 256, 0, s>>>((uint16_t*)logits, v, history_ids, n_ids, snapshot, penalty, logit_softcap);
    return launch_status();
}

namespace {
// Sampler.seedFor without a configured seed (Sampler.swift:311-323): the monotonic clock mixed
// with a process-wide counter, never zero.
uint64_t clock_seed() {
    static std::atomic<uint64_t> counter{0};
    timespec t{};
    clock_gettime(CLOCK_MONOTONIC, &t);
    const uint64_t c = counter.fetch_add(1, std::memory_order_relaxed) + 1;
    const uint64_t raw = ((uint64_t)t.tv_nsec + c) * 0x9E3779B97F4A7C15ull + (uint64_t)t.tv_sec;
    return raw == 0 ? 0x9E3779B97F4A7C15ull : raw;
}
}  // namespace

extern "C" int nvmai_hip_sampler_sample(nvmai_hip_ctx* ctx, nvmai_stream stream, void* logits, uint16_t* probs,
                                        uint32_t v, const int32_t* history_ids, uint32_t n_history,
                                        const nvmai_generation_config* config, int64_t position,
                                        float logit_softcap, int sampler_path, uint32_t* out_token,
                                        int* path_taken) {
    if (!ctx || !logits || !probs || !config || !out_token || v == 0) return NVMAI_ERR_INVALID_ARG;
    if (sampler_path != NVMAI_SAMPLER_TILED && sampler_path != NVMAI_SAMPLER_GENERIC) return NVMAI_ERR_INVALID_ARG;
    // GenerationConfig.validate (Sampler.swift:54-80), the parts the sampler reads
    const float T = config->temperature;
    if (!(T >= 0.0f) || T > 3.4e38f) return NVMAI_ERR_INVALID_ARG;
    if (config->top_k < 0 || config->top_k > 256) return NVMAI_ERR_INVALID_ARG;
    if (config->top_p < 0.0f || config->top_p > 1.0f || config->top_p != config->top_p) return NVMAI_ERR_INVALID_ARG;
    const bool has_k = config->top_k > 0, has_p = config->top_p > 0.0f;
    if (T > 0.0f && !has_k && has_p && config->top_p < 1.0f) return NVMAI_ERR_UNSUPPORTED;   // :76-79
    const bool penalty = config->repetition_penalty != 1.0f && n_history > 0;                // :180
    if (penalty) {
        const int rc = nvmai_hip_repetition_penalty(ctx, stream, logits, v, history_ids, n_history,
                                                    config->repetition_penalty, logit_softcap);
        if (rc) return rc;
    }
    // one front end serves both paths here: the tiled and the single-group softmax of the
    // reference agree to 1e-5 and differ only in how the work is cut
    int rc = nvmai_hip_softmax_tiled(ctx, stream, logits, v, probs, v, 1, v, logit_softcap);
    if (rc) return rc;
    const uint64_t seed = config->has_seed ? nvmai_sampler_seed_for(config->seed, position) : clock_seed();
    const float top_p = has_p ? config->top_p : 1.0f;
    if (sampler_path == NVMAI_SAMPLER_TILED && T > 0.0f && has_k && config->top_k <= 64 && v <= 262144) {   // :211-214
        rc = nvmai_hip_sample_topk64(ctx, stream, probs, v, 1, v, T, top_p, &seed, (uint32_t)config->top_k, out_token,
                                     nullptr);
    } else {
        const uint32_t pos = (uint32_t)position;
        rc = nvmai_hip_sample(ctx, stream, probs, v, 1, v, T, has_k ? (uint32_t)config->top_k : 0u, top_p, &seed, &pos,
                              out_token);
    }
    if (rc) return rc;
    if (path_taken)
        *path_taken = penalty ? NVMAI_SAMPLE_PATH_PENALTY : (T == 0.0f ? NVMAI_SAMPLE_PATH_GREEDY : NVMAI_SAMPLE_PATH_SAMPLED);
    return NVMAI_OK;
}
