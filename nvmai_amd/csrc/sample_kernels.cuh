// Softmax over the vocabulary and the tiled top-64 / generic samplers.  gfx950, wave64.
#pragma once

#include "common.cuh"

namespace nvmai {

constexpr int SOFTMAX_TILE = 4096;       // logit.metal:159
constexpr int SAMPLE_TILE = 1024;        // logit.metal:628-654
constexpr int SAMPLE_KEEP = 64;

__device__ __forceinline__ float softcap_value(float z, float softcap) {   // logit.metal:42-49
    return softcap <= 0.0f ? z : softcap * tanhf(z / softcap);
}

// (max, sum of exp) of two partial states, the empty state being (-inf, 0).
__device__ __forceinline__ void softmax_merge(float& m, float& d, float m2, float d2) {
    const float mn = fmaxf(m, m2);
    const float a = (m == -INFINITY) ? 0.0f : d * expf(m - mn);
    const float b = (m2 == -INFINITY) ? 0.0f : d2 * expf(m2 - mn);
    m = mn;
    d = a + b;
}

__device__ __forceinline__ void block_softmax_merge(float& m, float& d, float* lds) {
    // wave butterfly, then the four waves through LDS; every thread ends with the block result
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float m2 = shfl_xor_f(m, off), d2 = shfl_xor_f(d, off);
        softmax_merge(m, d, m2, d2);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { lds[2 * wave] = m; lds[2 * wave + 1] = d; }
    __syncthreads();
    m = lds[0]; d = lds[1];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) softmax_merge(m, d, lds[2 * w], lds[2 * w + 1]);
    __syncthreads();
}

// Stage 1 (logit.metal:155-200): per 4096-entry tile the running (max, sum exp).
template <int ACT>
__global__ __launch_bounds__(256) void softmax_stage1_kernel(const void* logits, uint32_t v, uint32_t row_stride,
                                                            float softcap, float* tile_max, float* tile_sum,
                                                            uint32_t tiles) {
    __shared__ float lds[8];
    const uint32_t tile = blockIdx.x, row = blockIdx.y;
    const uint16_t* z = (const uint16_t*)logits + (size_t)row * row_stride;
    const uint32_t base = tile * SOFTMAX_TILE, end = min(base + SOFTMAX_TILE, v);
    float m = -INFINITY, d = 0.0f;
    for (uint32_t i = base + threadIdx.x; i < end; i += 256) {
        const float x = softcap_value(act_to_f32<ACT>(z[i]), softcap);
        softmax_merge(m, d, x, 1.0f);
    }
    block_softmax_merge(m, d, lds);
    if (threadIdx.x == 0) { tile_max[(size_t)row * tiles + tile] = m; tile_sum[(size_t)row * tiles + tile] = d; }
}

// Merge + normalize (logit.metal:202-257): every block folds the tile partials again
// (a few dozen values), then writes probs = exp(z - max) * (1 / sum) as fp16.
template <int ACT>
__global__ __launch_bounds__(256) void softmax_normalize_kernel(const void* logits, uint32_t v, uint32_t row_stride,
                                                               float softcap, const float* tile_max,
                                                               const float* tile_sum, uint32_t tiles,
                                                               uint16_t* probs, uint32_t probs_stride) {
    __shared__ float lds[8];
    const uint32_t row = blockIdx.y;
    float m = -INFINITY, d = 0.0f;
    for (uint32_t t = threadIdx.x; t < tiles; t += 256)
        softmax_merge(m, d, tile_max[(size_t)row * tiles + t], tile_sum[(size_t)row * tiles + t]);
    block_softmax_merge(m, d, lds);
    const float inv = d > 0.0f ? 1.0f / d : 0.0f;
    const uint16_t* z = (const uint16_t*)logits + (size_t)row * row_stride;
    uint16_t* out = probs + (size_t)row * probs_stride;
    const uint32_t base = blockIdx.x * SOFTMAX_TILE, end = min(base + SOFTMAX_TILE, v);
    for (uint32_t i = base + threadIdx.x; i < end; i += 256)
        out[i] = f32_to_f16(expf(softcap_value(act_to_f32<ACT>(z[i]), softcap) - m) * inv);
}

// ---- sampling ------------------------------------------------------------------------
constexpr int SAMPLE_MAX_ROWS = 32;
struct SeedArray { uint64_t s[SAMPLE_MAX_ROWS]; };   // one PRNG seed per row, passed by value

__device__ __forceinline__ uint64_t xorshift64star(uint64_t& s) {        // logit.metal:280-285
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s * 2685821657736338717ull;
}

__device__ __forceinline__ float uniform01(uint64_t& s) {                // logit.metal:287-292
    return (float)(uint32_t)(xorshift64star(s) >> 40) * (1.0f / 16777216.0f);
}

// Total order "better(a, b) = a.v > b.v || (a.v == b.v && a.i < b.i)" (logit.metal:590-594)
// as one unsigned compare: high word = order-preserving image of the float, low word = ~index.
__device__ __forceinline__ uint64_t sample_key(float v, uint32_t idx) {
    uint32_t u = __float_as_uint(v);
    u ^= (u >> 31) ? 0xFFFFFFFFu : 0x80000000u;
    return ((uint64_t)u << 32) | (uint32_t)~idx;
}
__device__ __forceinline__ float key_value(uint64_t k) {
    uint32_t u = (uint32_t)(k >> 32);
    u ^= (u >> 31) ? 0x80000000u : 0xFFFFFFFFu;
    return __uint_as_float(u);
}
__device__ __forceinline__ uint32_t key_index(uint64_t k) { return ~(uint32_t)k; }

// The reference sorts every 1024-entry tile with a bitonic network in threadgroup memory and
// keeps the first 64 (logit.metal:596-626).  Only those 64 matter, and the comparator is a total
// order, so any exact selection gives the same keys in the same order.  Here each wave sorts 256
// keys held in registers (key i = reg * 64 + lane; strides below 64 are lane exchanges, 64 and
// 128 are register swaps: no barriers), the four waves' best 64 meet in LDS, and wave 0 sorts
// those 256 once more.
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask) {
    const uint32_t lo = shfl_xor_u((uint32_t)v, mask), hi = shfl_xor_u((uint32_t)(v >> 32), mask);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ void wave_sort256_desc(uint64_t k[4], int lane) {
#pragma unroll
    for (int width = 2; width <= 256; width <<= 1) {
#pragma unroll
        for (int stride = width >> 1; stride > 0; stride >>= 1) {
            if (stride >= 64) {
                const int rs = stride >> 6;                        // partner register = r ^ rs
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (r & rs) continue;
                    const bool desc = (((r << 6) | lane) & width) == 0;
                    const uint64_t a = k[r], b = k[r ^ rs];
                    const bool swap = desc ? (b > a) : (a > b);
                    k[r] = swap ? b : a;
                    k[r ^ rs] = swap ? a : b;
                }
            } else {
                const bool lower = (lane & stride) == 0;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool desc = (((r << 6) | lane) & width) == 0;
                    const uint64_t a = k[r], b = shfl_xor_u64(a, stride);
                    const bool take_max = desc == lower;
                    k[r] = take_max ? (a > b ? a : b) : (a > b ? b : a);
                }
            }
        }
    }
}

// The best SAMPLE_KEEP of the block's 1024 keys (mine[r] = key r * 256 + thread), descending,
// returned in lanes 0..63 of wave 0 (`valid` there); `cand` is 256 keys of LDS.
__device__ __forceinline__ uint64_t tile_top64(uint64_t mine[4], uint64_t* cand, bool& valid) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    wave_sort256_desc(mine, lane);
    cand[wave * 64 + lane] = mine[0];                             // sorted keys 0..63 of this wave
    __syncthreads();
    valid = wave == 0;
    uint64_t k[4] = {0, 0, 0, 0};
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) k[r] = cand[r * 64 + lane];
        wave_sort256_desc(k, lane);
    }
    return k[0];
}

// Stage 1 (logit.metal:628-654): top 64 of each 1024-entry tile of the fp16 probabilities.
__global__ __launch_bounds__(256) void sample_topk64_stage1_kernel(const uint16_t* probs, uint32_t v,
                                                                   uint32_t probs_stride, uint64_t* out,
                                                                   uint32_t out_row_stride) {
    __shared__ uint64_t cand[256];
    const uint32_t row = blockIdx.y, base = blockIdx.x * SAMPLE_TILE;
    const uint16_t* p = probs + (size_t)row * probs_stride;
    uint64_t mine[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t src = base + r * 256 + threadIdx.x;
        mine[r] = src < v ? sample_key(f16_to_f32(p[src]), src) : sample_key(-INFINITY, 0xFFFFFFFFu);
    }
    bool valid;
    const uint64_t best = tile_top64(mine, cand, valid);
    if (valid) out[(size_t)row * out_row_stride + blockIdx.x * SAMPLE_KEEP + threadIdx.x] = best;
}

// Reduce (logit.metal:656-682): top 64 of each 1024 surviving candidates.
__global__ __launch_bounds__(256) void sample_topk64_reduce_kernel(const uint64_t* in, uint32_t count,
                                                                   uint32_t in_row_stride, uint64_t* out,
                                                                   uint32_t out_row_stride) {
    __shared__ uint64_t cand[256];
    const uint32_t row = blockIdx.y, base = blockIdx.x * SAMPLE_TILE;
    uint64_t mine[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t src = base + r * 256 + threadIdx.x;
        mine[r] = src < count ? in[(size_t)row * in_row_stride + src] : sample_key(-INFINITY, 0xFFFFFFFFu);
    }
    bool valid;
    const uint64_t best = tile_top64(mine, cand, valid);
    if (valid) out[(size_t)row * out_row_stride + blockIdx.x * SAMPLE_KEEP + threadIdx.x] = best;
}

// Selection over the sorted candidates (logit.metal:704-757 == :517-571): cap at k,
// top-p cut on the cumulative mass, p^(1/T), inverse-CDF draw with xorshift64*.
__device__ inline uint32_t sample_select(float* val, const uint32_t* idx, uint32_t kept, float temperature,
                                         float top_p, uint64_t seed, uint32_t fallback) {
    if (top_p > 0.0f && top_p < 1.0f) {
        float cum = 0.0f;
        uint32_t cut = kept;
        for (uint32_t i = 0; i < kept; ++i) {
            cum = __fadd_rn(cum, val[i]);
            if (cum >= top_p) { cut = i + 1; break; }
        }
        kept = cut;
    }
    const float inv_t = __fdiv_rn(1.0f, temperature);
    if (temperature != 1.0f)
        for (uint32_t i = 0; i < kept; ++i) val[i] = powf(val[i], inv_t);
    float surviving = 0.0f;
    for (uint32_t i = 0; i < kept; ++i) surviving = __fadd_rn(surviving, val[i]);
    uint64_t rng = seed;
    (void)xorshift64star(rng);
    const float u = __fmul_rn(uniform01(rng), surviving);
    float run = 0.0f;
    uint32_t picked = fallback;
    for (uint32_t i = 0; i < kept; ++i) {
        run = __fadd_rn(run, val[i]);
        if (u <= run) { picked = idx[i]; break; }
    }
    return picked;
}

// Final (logit.metal:684-758).  seeds: one per row.  top64 (optional): the 64 sorted
// candidates per row as (value bits, index) pairs.
__global__ __launch_bounds__(256) void sample_topk64_final_kernel(const uint64_t* in, uint32_t count,
                                                                  uint32_t in_row_stride, float temperature,
                                                                  float top_p, SeedArray seeds,
                                                                  uint32_t top_k, uint32_t* out_token,
                                                                  uint32_t* top64) {
    __shared__ uint64_t cand[256];
    __shared__ float val[SAMPLE_KEEP];
    __shared__ uint32_t idx[SAMPLE_KEEP];
    const uint32_t row = blockIdx.x;
    uint64_t mine[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t i = r * 256 + threadIdx.x;
        mine[r] = i < count ? in[(size_t)row * in_row_stride + i] : sample_key(-INFINITY, 0xFFFFFFFFu);
    }
    bool valid;
    const uint64_t best = tile_top64(mine, cand, valid);
    if (valid) {
        val[threadIdx.x] = key_value(best);
        idx[threadIdx.x] = key_index(best);
        if (top64) {
            top64[((size_t)row * SAMPLE_KEEP + threadIdx.x) * 2] = __float_as_uint(val[threadIdx.x]);
            top64[((size_t)row * SAMPLE_KEEP + threadIdx.x) * 2 + 1] = idx[threadIdx.x];
        }
    }
    __syncthreads();
    if (threadIdx.x >= 64) return;
    // wave 0: the candidates' p^(1/T) in parallel (the same function on other lanes: the same
    // bits), every running sum by lane 0 in candidate order as the reference's single thread does
    __shared__ float powed[SAMPLE_KEEP];
    const float inv_t = __fdiv_rn(1.0f, temperature);
    powed[threadIdx.x] = temperature != 1.0f ? powf(val[threadIdx.x], inv_t) : val[threadIdx.x];
    __builtin_amdgcn_wave_barrier();
    if (threadIdx.x == 0) {
        uint32_t kept = 0;
        while (kept < SAMPLE_KEEP && idx[kept] != 0xFFFFFFFFu && isfinite(val[kept])) kept++;
        kept = min(kept, max(1u, top_k));
        if (top_p > 0.0f && top_p < 1.0f) {
            float cum = 0.0f;
            uint32_t cut = kept;
            for (uint32_t i = 0; i < kept; ++i) {
                cum = __fadd_rn(cum, val[i]);
                if (cum >= top_p) { cut = i + 1; break; }
            }
            kept = cut;
        }
        float surviving = 0.0f;
        for (uint32_t i = 0; i < kept; ++i) surviving = __fadd_rn(surviving, powed[i]);
        uint64_t rng = seeds.s[row];
        (void)xorshift64star(rng);
        const float u = __fmul_rn(uniform01(rng), surviving);
        float run = 0.0f;
        uint32_t picked = idx[0];
        for (uint32_t i = 0; i < kept; ++i) {
            run = __fadd_rn(run, powed[i]);
            if (u <= run) { picked = idx[i]; break; }
        }
        out_token[row] = picked;
    }
}

// Generic sampler (logit.metal:315-585): greedy argmax at temperature <= 0, else k argmax
// passes over the vocabulary (k <= 256), then the same selection.  One block per row.
__global__ __launch_bounds__(256) void sample_generic_kernel(const uint16_t* probs, uint32_t v,
                                                             uint32_t probs_stride, float temperature,
                                                             uint32_t top_k, float top_p, SeedArray seeds,
                                                             uint32_t* out_token) {
    __shared__ uint64_t wave_best[4];
    __shared__ float val[256];
    __shared__ uint32_t idx[256];
    const uint32_t row = blockIdx.x;
    const uint16_t* p = probs + (size_t)row * probs_stride;
    uint32_t k = temperature <= 0.0f ? 1u : (top_k == 0 ? v : top_k);
    k = min(min(k, 256u), v);
    uint64_t prev = ~0ull;               // every later pass takes the best key below the previous one
    for (uint32_t slot = 0; slot < k; ++slot) {
        uint64_t best = 0;
        for (uint32_t i = threadIdx.x; i < v; i += 256) {
            const float pv = f16_to_f32(p[i]);
            if (!(pv > -INFINITY)) continue;                 // the kernel's `p > best_v` never takes -inf or NaN
            const uint64_t key = sample_key(pv, i);
            if (key < prev && key > best) best = key;
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const uint32_t lo = shfl_xor_u((uint32_t)best, off), hi = shfl_xor_u((uint32_t)(best >> 32), off);
            const uint64_t o = ((uint64_t)hi << 32) | lo;
            best = o > best ? o : best;
        }
        if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
        __syncthreads();
        best = max(max(wave_best[0], wave_best[1]), max(wave_best[2], wave_best[3]));
        if (threadIdx.x == 0) {
            val[slot] = best ? key_value(best) : -INFINITY;
            idx[slot] = best ? key_index(best) : 0xFFFFFFFFu;
        }
        prev = best ? best : 0;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (temperature <= 0.0f) { out_token[row] = idx[0]; return; }
        uint32_t kept = 0;
        while (kept < k && idx[kept] < v && isfinite(val[kept])) kept++;
        out_token[row] = sample_select(val, idx, kept, temperature, top_p, seeds.s[row], kept > 0 ? idx[0] : 0u);
    }
}

// Gumbel-max draw the reference takes when neither top-k nor top-p is set (logit.metal:296-313,
// 391-429): argmax_i(log(p_i) / T + g_i), g_i = -log(-log(u_i)), u_i from SplitMix64 of
// (seed, position, i).  Logarithms in double, rounded to float once per step, so that scores
// are the same bits on every device.  GUMBEL_BLOCKS blocks per row; the last one to finish
// folds the block winners (highest score, lowest index among equals).
constexpr int GUMBEL_BLOCKS = 64;
struct PosArray { uint32_t p[SAMPLE_MAX_ROWS]; };

__device__ __forceinline__ float gumbel_for(uint64_t seed, uint32_t position, uint32_t row) {
    uint64_t x = seed ^ ((uint64_t)position * 0xD2B74407B1CE6E93ull) ^ (uint64_t)row;
    x = x + 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x = x ^ (x >> 31);
    const float u = __fmul_rn(__fadd_rn((float)(uint32_t)(x >> 40), 0.5f), 1.0f / 16777216.0f);
    const float inner = (float)log((double)u);
    return -(float)log((double)(-inner));
}

__global__ __launch_bounds__(256) void sample_gumbel_kernel(const uint16_t* probs, uint32_t v, uint32_t probs_stride,
                                                            float temperature, SeedArray seeds, PosArray positions,
                                                            uint64_t* block_best, uint32_t* tickets,
                                                            uint32_t* out_token) {
    __shared__ uint64_t wave_best[4];
    __shared__ bool last;
    const uint32_t row = blockIdx.y;
    const uint16_t* p = probs + (size_t)row * probs_stride;
    const float inv_t = __fdiv_rn(1.0f, temperature);
    uint64_t best = 0;                                   // keys of real candidates are never 0
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < v; i += GUMBEL_BLOCKS * 256) {
        const float pv = f16_to_f32(p[i]);
        if (!(pv > 0.0f)) continue;
        const float sc = __fadd_rn(__fmul_rn(inv_t, (float)log((double)pv)), gumbel_for(seeds.s[row], positions.p[row], i));
        const uint64_t key = sample_key(sc, i);
        best = key > best ? key : best;
    }
    auto fold = [&](uint64_t b) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const uint32_t lo = shfl_xor_u((uint32_t)b, off), hi = shfl_xor_u((uint32_t)(b >> 32), off);
            const uint64_t o = ((uint64_t)hi << 32) | lo;
            b = o > b ? o : b;
        }
        return b;
    };
    best = fold(best);
    if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        best = max(max(wave_best[0], wave_best[1]), max(wave_best[2], wave_best[3]));
        block_best[(size_t)row * GUMBEL_BLOCKS + blockIdx.x] = best;
        __threadfence();
        last = atomicAdd(&tickets[row], 1u) == GUMBEL_BLOCKS - 1;
    }
    __syncthreads();
    if (!last) return;
    __threadfence();
    uint64_t b = threadIdx.x < GUMBEL_BLOCKS ? block_best[(size_t)row * GUMBEL_BLOCKS + threadIdx.x] : 0;
    if (threadIdx.x < 64) {
        b = fold(b);
        if (threadIdx.x == 0) {
            out_token[row] = b ? key_index(b) : 0u;      // nothing eligible: the reference falls back to 0
            tickets[row] = 0;                            // ready for the next call
        }
    }
}

}  // namespace nvmai
