// Softmax over the vocabulary and the tiled top-64 / generic samplers.  gfx950, wave64.
#pragma once

#include "common.hpp"

namespace nvmai {

constexpr int SOFTMAX_TILE = 4096;       // logit.metal:159
constexpr int SAMPLE_TILE = 1024;        // logit.metal:628-654
constexpr int SAMPLE_KEEP = 64;

// softcap * tanh(z / softcap) (logit.metal:42-49) with tanh(t) = 1 - 2 / (exp(2 t) + 1) on the
// hardware exponential, as the reference computes it with its fast-math tanh: the absolute error
// is a few 1e-7 of the cap, far below what an fp16 probability resolves.
__device__ __forceinline__ float softcap_value(float z, float softcap) {
    if (softcap <= 0.0f) return z;
    const float t = fminf(fmaxf(__fdividef(z, softcap), -15.0f), 15.0f);
    return softcap * (1.0f - __fdividef(2.0f, __expf(2.0f * t) + 1.0f));
}

// (max, sum of exp) of two partial states, the empty state being (-inf, 0).
__device__ __forceinline__ void softmax_merge(float& m, float& d, float m2, float d2) {
    const float mn = fmaxf(m, m2);
    const float a = (m == -INFINITY) ? 0.0f : d * expf(m - mn);
    const float b = (m2 == -INFINITY) ? 0.0f : d2 * expf(m2 - mn);
    m = mn;
    d = a + b;
}

// Every thread ends with the block's state: the maximum first (max reductions only), then each
// state's sum rescaled to it once, then plain sums.  Equal to folding softmax_merge over the
// states up to the rounding of the additions.
__device__ __forceinline__ void block_softmax_merge(float& m, float& d, float* lds) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float wm = wave_max_f32(m);
    if (lane == 0) lds[wave] = wm;
    __syncthreads();
    float bm = lds[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) bm = fmaxf(bm, lds[w]);
    const float scaled = (m == -INFINITY) ? 0.0f : d * __expf(m - bm);
    const float ws = wave_sum_bcast(scaled);
    if (lane == 0) lds[4 + wave] = ws;
    __syncthreads();
    float bd = lds[4];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) bd += lds[4 + w];
    __syncthreads();
    m = bm;
    d = bd;
}

// A thread's 16 entries of a 4096-entry tile, softcap applied, -inf past the end of the row:
// two 16-byte loads (entries 8 t .. 8 t + 7 of each half of the tile) where the tile is whole
// and the row 16-byte aligned, element loads otherwise.  at[j] = position of x[j] in the row.
constexpr int SOFTMAX_PER_THREAD = SOFTMAX_TILE / 256;

template <int ACT>
__device__ __forceinline__ bool softmax_load(const uint16_t* z, uint32_t base, uint32_t v, float softcap, float* x) {
    const bool vec = (reinterpret_cast<uintptr_t>(z + base) & 15u) == 0 && base + SOFTMAX_TILE <= v;
    if (vec) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint4 q = *reinterpret_cast<const uint4*>(z + base + h * (SOFTMAX_TILE / 2) + 8 * threadIdx.x);
            act2_to_f32<ACT>(q.x, x[8 * h], x[8 * h + 1]);
            act2_to_f32<ACT>(q.y, x[8 * h + 2], x[8 * h + 3]);
            act2_to_f32<ACT>(q.z, x[8 * h + 4], x[8 * h + 5]);
            act2_to_f32<ACT>(q.w, x[8 * h + 6], x[8 * h + 7]);
        }
#pragma unroll
        for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) x[j] = softcap_value(x[j], softcap);
    } else {
#pragma unroll
        for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) {
            const uint32_t i = base + (j / 8) * (SOFTMAX_TILE / 2) + 8 * threadIdx.x + (j % 8);
            x[j] = i < v ? softcap_value(act_to_f32<ACT>(z[i]), softcap) : -INFINITY;
        }
    }
    return vec;
}

// Stage 1 (logit.metal:155-200): per 4096-entry tile the (max, sum exp) state.  A thread takes
// the maximum of its entries first and then one exponential per entry; states merge as the
// reference's recurrence merges them.
template <int ACT>
__global__ __launch_bounds__(256) void softmax_stage1_kernel(const void* logits, uint32_t v, uint32_t row_stride,
                                                            float softcap, float* tile_max, float* tile_sum,
                                                            uint32_t tiles) {
    __shared__ float lds[8];
    const uint32_t tile = blockIdx.x, row = blockIdx.y;
    const uint16_t* z = (const uint16_t*)logits + (size_t)row * row_stride;
    float x[SOFTMAX_PER_THREAD];
    softmax_load<ACT>(z, tile * SOFTMAX_TILE, v, softcap, x);
    float m = -INFINITY, d = 0.0f;
#pragma unroll
    for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) m = fmaxf(m, x[j]);
    if (m != -INFINITY) {
#pragma unroll
        for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) d += __expf(x[j] - m);   // exp(-inf) = 0 past the end
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
    const uint16_t* z = (const uint16_t*)logits + (size_t)row * row_stride;
    const uint32_t base = blockIdx.x * SOFTMAX_TILE;
    float x[SOFTMAX_PER_THREAD];
    const bool vec = softmax_load<ACT>(z, base, v, softcap, x);   // in flight while the partials merge
    float m = -INFINITY, d = 0.0f;
    for (uint32_t t = threadIdx.x; t < tiles; t += 256)
        softmax_merge(m, d, tile_max[(size_t)row * tiles + t], tile_sum[(size_t)row * tiles + t]);
    block_softmax_merge(m, d, lds);
    const float inv = d > 0.0f ? 1.0f / d : 0.0f;
    uint16_t* out = probs + (size_t)row * probs_stride;
    uint16_t pr[SOFTMAX_PER_THREAD];
#pragma unroll
    for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) pr[j] = f32_to_f16(__expf(x[j] - m) * inv);
    if (vec && (reinterpret_cast<uintptr_t>(out + base) & 15u) == 0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint4 q;
            q.x = pr[8 * h] | ((uint32_t)pr[8 * h + 1] << 16);
            q.y = pr[8 * h + 2] | ((uint32_t)pr[8 * h + 3] << 16);
            q.z = pr[8 * h + 4] | ((uint32_t)pr[8 * h + 5] << 16);
            q.w = pr[8 * h + 6] | ((uint32_t)pr[8 * h + 7] << 16);
            *reinterpret_cast<uint4*>(out + base + h * (SOFTMAX_TILE / 2) + 8 * threadIdx.x) = q;
        }
    } else {
#pragma unroll
        for (int j = 0; j < SOFTMAX_PER_THREAD; ++j) {
            const uint32_t i = base + (j / 8) * (SOFTMAX_TILE / 2) + 8 * threadIdx.x + (j % 8);
            if (i < v) out[i] = pr[j];
        }
    }
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
// order, so any exact selection gives the same keys in the same order.  Here a wave holds 256
// keys in four registers and selects instead of sorting: each register is sorted over the 64
// lanes (even registers descending, odd ones ascending), the element-wise larger of a
// descending and an ascending run holds the best 64 of their 128 as a bitonic run, which six
// more exchange steps sort; twice more and the best 64 of the 256 stand sorted in one register.
// No barriers, no LDS.  The four waves' best 64 meet in LDS and wave 0 selects once more, from
// runs that are sorted already.  K: 64-bit (value, ~index) keys, or 32-bit keys where a tile's
// value and position fit (half the exchange traffic, single-instruction compares).
// The value of lane ^ stride.  Distances 1, 2, 4 and 8 stay inside a row of 16 lanes and are data
// parallel moves of the vector pipe (quad permutes, row rotations: a rotation by 8 is the
// exchange itself, at 4 the lane takes the rotation that reaches its partner); 16 and 32 go
// through the LDS crossbar.  `stride` is a constant wherever this is inlined.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ uint32_t lane_xor_u32(uint32_t v, int stride, int lane) {
    if (stride == 1) return dpp_u32<0xB1>(v);                      // quad_perm [1,0,3,2]
    if (stride == 2) return dpp_u32<0x4E>(v);                      // quad_perm [2,3,0,1]
    if (stride == 8) return dpp_u32<0x128>(v);                     // row_ror:8
    if (stride == 4) {
        const uint32_t from_below = dpp_u32<0x124>(v);             // row_ror:4: lane i <- lane i - 4
        const uint32_t from_above = dpp_u32<0x12C>(v);             // row_ror:12: lane i <- lane i + 4
        return (lane & 4) ? from_below : from_above;
    }
    return shfl_xor_u(v, stride);
}
// 32-bit keys: the many small tiles of the first stage keep every vector pipe busy, and the
// crossbar takes the exchange off it.  64-bit keys: a few blocks per row whose chain of
// dependent exchanges is what takes the time, and the in-row moves are the shorter way.
__device__ __forceinline__ uint32_t shfl_xor_key(uint32_t v, int stride, int) { return shfl_xor_u(v, stride); }
__device__ __forceinline__ uint64_t shfl_xor_key(uint64_t v, int stride, int lane) {
    const uint32_t lo = lane_xor_u32((uint32_t)v, stride, lane), hi = lane_xor_u32((uint32_t)(v >> 32), stride, lane);
    return ((uint64_t)hi << 32) | lo;
}

// One exchange step at lane distance `stride`: lanes of a pair keep the larger key in the lower
// lane where `desc`, in the upper lane otherwise.
template <typename K>
__device__ __forceinline__ K lane_exchange(K a, int lane, int stride, bool desc) {
    const K b = shfl_xor_key(a, stride, lane);
    const bool lower = (lane & stride) == 0;
    const K hi = a > b ? a : b, lo = a > b ? b : a;
    return desc == lower ? hi : lo;
}

// A bitonic run over the 64 lanes -> sorted (descending or ascending).
template <typename K>
__device__ __forceinline__ K lane_merge64(K k, int lane, bool desc) {
#pragma unroll
    for (int stride = 32; stride > 0; stride >>= 1) k = lane_exchange(k, lane, stride, desc);
    return k;
}

// Any 64 keys over the lanes -> sorted.
template <typename K>
__device__ __forceinline__ K lane_sort64(K k, int lane, bool desc) {
#pragma unroll
    for (int width = 2; width < 64; width <<= 1) {
        const bool block_desc = ((lane & width) == 0) == desc;
#pragma unroll
        for (int stride = width >> 1; stride > 0; stride >>= 1) k = lane_exchange(k, lane, stride, block_desc);
    }
    return lane_merge64(k, lane, desc);
}

// The best 64 of the wave's 256 keys, descending over the lanes.  sorted: k[0], k[2] already
// descend and k[1], k[3] already ascend over the lanes.
template <typename K>
__device__ __forceinline__ K wave_top64(K k[4], int lane, bool sorted) {
    if (!sorted) {
#pragma unroll
        for (int r = 0; r < 4; ++r) k[r] = lane_sort64(k[r], lane, (r & 1) == 0);
    }
    const K m0 = lane_merge64(k[0] > k[1] ? k[0] : k[1], lane, true);
    const K m1 = lane_merge64(k[2] > k[3] ? k[2] : k[3], lane, false);
    return lane_merge64(m0 > m1 ? m0 : m1, lane, true);
}

// The best SAMPLE_KEEP of the block's 1024 keys (any assignment of keys to threads and
// registers), descending, returned in lanes 0..63 of wave 0 (`valid` there); `cand` is 256 keys
// of LDS.
template <typename K>
__device__ __forceinline__ K tile_top64(K mine[4], K* cand, bool& valid) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    cand[wave * 64 + lane] = wave_top64(mine, lane, false);
    __syncthreads();
    valid = wave == 0;
    K best = 0;
    if (wave == 0) {
        K k[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) k[r] = cand[r * 64 + ((r & 1) ? 63 - lane : lane)];
        best = wave_top64(k, lane, true);
    }
    return best;
}

// Stage 1 (logit.metal:628-654): top 64 of each 1024-entry tile of the fp16 probabilities.
// Inside a tile a 32-bit key orders like the 64-bit one: the order-preserving image of the
// fp16 bits above 1024 - position (so that the earlier of two equal values wins and every real
// entry beats the zero key of the padding past the end of the row).
__device__ __forceinline__ uint32_t tile_key(uint16_t h, uint32_t pos) {
    const uint32_t image = h ^ ((h >> 15) ? 0xFFFFu : 0x8000u);
    return (image << 16) | (uint32_t)(SAMPLE_TILE - pos);
}

__global__ __launch_bounds__(256) void sample_topk64_stage1_kernel(const uint16_t* probs, uint32_t v,
                                                                   uint32_t probs_stride, uint64_t* out,
                                                                   uint32_t out_row_stride) {
    __shared__ uint32_t cand[256];
    const uint32_t row = blockIdx.y, base = blockIdx.x * SAMPLE_TILE;
    const uint16_t* p = probs + (size_t)row * probs_stride;
    uint32_t mine[4];
    const uint32_t first = 4 * threadIdx.x;                       // the thread's four neighbours
    if (((reinterpret_cast<uintptr_t>(p + base) & 7u) == 0) && base + SAMPLE_TILE <= v) {
        const uint2 q = *reinterpret_cast<const uint2*>(p + base + first);
        mine[0] = tile_key((uint16_t)(q.x & 0xFFFFu), first);
        mine[1] = tile_key((uint16_t)(q.x >> 16), first + 1);
        mine[2] = tile_key((uint16_t)(q.y & 0xFFFFu), first + 2);
        mine[3] = tile_key((uint16_t)(q.y >> 16), first + 3);
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[r] = base + first + r < v ? tile_key(p[base + first + r], first + r) : 0u;
    }
    bool valid;
    const uint32_t best = tile_top64(mine, cand, valid);
    if (valid) {
        uint64_t key = sample_key(-INFINITY, 0xFFFFFFFFu);        // fewer than 64 entries in the tile
        if (best) {
            const uint32_t image = best >> 16;
            const uint16_t h = (uint16_t)(image ^ ((image >> 15) ? 0x8000u : 0xFFFFu));
            key = sample_key(f16_to_f32(h), base + SAMPLE_TILE - (best & 0xFFFFu));
        }
        out[(size_t)row * out_row_stride + blockIdx.x * SAMPLE_KEEP + threadIdx.x] = key;
    }
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
    const uint32_t row = blockIdx.x;
    uint64_t mine[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t i = r * 256 + threadIdx.x;
        mine[r] = i < count ? in[(size_t)row * in_row_stride + i] : sample_key(-INFINITY, 0xFFFFFFFFu);
    }
    bool valid;
    const uint64_t best = tile_top64(mine, cand, valid);
    if (!valid) return;                                            // wave 0 goes on: lane = candidate
    const float val = key_value(best);
    const uint32_t idx = key_index(best);
    if (top64) {
        top64[((size_t)row * SAMPLE_KEEP + threadIdx.x) * 2] = __float_as_uint(val);
        top64[((size_t)row * SAMPLE_KEEP + threadIdx.x) * 2 + 1] = idx;
    }
    // p^(1/T) of every candidate in parallel (the same function on other lanes: the same bits).
    // The running sums are the reference's single-thread loops, candidate after candidate in
    // order: every lane carries the same sum and takes candidate i from lane i, so that a step
    // is a lane read and an addition with no memory in between; "stop at the first i that ..."
    // becomes "remember the first i that ...".
    const float inv_t = __fdiv_rn(1.0f, temperature);
    const float powed = temperature != 1.0f ? powf(val, inv_t) : val;
    const unsigned long long usable = __ballot(idx != 0xFFFFFFFFu && isfinite(val));
    uint32_t kept = ~usable ? (uint32_t)__builtin_ctzll(~usable) : (uint32_t)SAMPLE_KEEP;
    kept = min(kept, max(1u, top_k));
    if (top_p > 0.0f && top_p < 1.0f) {
        float cum = 0.0f;
        uint32_t cut = kept;
        bool found = false;
#pragma unroll
        for (int i = 0; i < SAMPLE_KEEP; ++i) {
            cum = __fadd_rn(cum, readlane_f(val, i));
            const bool hit = !found && (uint32_t)i < kept && cum >= top_p;
            cut = hit ? (uint32_t)i + 1u : cut;
            found = found || hit;
        }
        kept = cut;
    }
    float surviving = 0.0f;
#pragma unroll
    for (int i = 0; i < SAMPLE_KEEP; ++i)
        surviving = (uint32_t)i < kept ? __fadd_rn(surviving, readlane_f(powed, i)) : surviving;
    uint64_t rng = seeds.s[row];
    (void)xorshift64star(rng);
    const float u = __fmul_rn(uniform01(rng), surviving);
    float run = 0.0f;
    uint32_t picked = (uint32_t)__builtin_amdgcn_readlane((int)idx, 0);
    bool found = false;
#pragma unroll
    for (int i = 0; i < SAMPLE_KEEP; ++i) {
        run = __fadd_rn(run, readlane_f(powed, i));
        const bool hit = !found && (uint32_t)i < kept && u <= run;
        picked = hit ? (uint32_t)__builtin_amdgcn_readlane((int)idx, i) : picked;
        found = found || hit;
    }
    if (threadIdx.x == 0) out_token[row] = picked;
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
        // greedy: with no value above -inf (all NaN or -inf) the reference's reduction ends at index 0
        // (logit.metal:340-382: every lane starts at best_i = 0), never at an out-of-range id
        if (temperature <= 0.0f) { out_token[row] = idx[0] == 0xFFFFFFFFu ? 0u : idx[0]; return; }
        uint32_t kept = 0;
        while (kept < k && idx[kept] < v && isfinite(val[kept])) kept++;
        out_token[row] = sample_select(val, idx, kept, temperature, top_p, seeds.s[row], kept > 0 ? idx[0] : 0u);
    }
}

// Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293) on the device, one thread per history
// entry, in two launches.  The reference walks the distinct ids of its history dictionary; a list may
// hold an id many times.  The first launch copies the logit of every entry into a snapshot; the second
// writes the penalised value computed from the snapshot: entries with the same id write the same bits,
// so repeats need no search for an earlier occurrence (that search was a chain of up to n dependent
// reads in the last thread: quadratic in the history, which reaches 128K tokens).  Without a softcap
// the new logit is one IEEE division or product, rounded to the activation type.
__global__ __launch_bounds__(256) void repetition_penalty_gather_kernel(const uint16_t* logits, uint32_t v, const int32_t* ids,
                                                                        uint32_t n_ids, uint16_t* snapshot) {
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= n_ids) return;
    const int32_t id = ids[j];
    snapshot[j] = (id < 0 || (uint32_t)id >= v) ? (uint16_t)0 : logits[id];
}

template <int ACT>
__global__ __launch_bounds__(256) void repetition_penalty_kernel(uint16_t* logits, uint32_t v, const int32_t* ids,
                                                                 uint32_t n_ids, const uint16_t* snapshot, float penalty,
                                                                 float softcap) {
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= n_ids) return;
    const int32_t id = ids[j];
    if (id < 0 || (uint32_t)id >= v) return;
    const float z = act_to_f32<ACT>(snapshot[j]);
    float out;
    if (softcap > 0.0f) {
        const float capped = softcap * tanhf(z / softcap);
        const float pen = capped > 0.0f ? capped / penalty : capped * penalty;
        const float limit = softcap * 0.9999f;
        const float clamped = fmaxf(fminf(pen, limit), -limit);
        out = softcap * atanhf(clamped / softcap);
    } else {
        out = z > 0.0f ? z / penalty : z * penalty;
    }
    logits[id] = f32_to_act<ACT>(out);
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
