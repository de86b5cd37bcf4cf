// Prefill side of the MoE path: token-expert pair records, the permutation / histogram by
// expert, the grouped expert GEMMs (dequant to bf16 tiles in LDS + MFMA) and the rank-order
// combine.  gfx950, wave64.
#pragma once

#include "common.hpp"

namespace nvmai {

// PrefillTokenExpertPair (PrefillRouter.swift:5-28): 16 bytes, fields at 0/4/8/12.
struct PrefillPair { uint32_t token, expert, rank, weight_bits; };
struct PrefillGroup { uint32_t expert, pair_start, pair_count; };                 // PrefillMoEGroup
struct PrefillTile { uint32_t group_start, group_count, pair_start, pair_count; }; // PrefillMoETile

constexpr int GROUP_CHUNK = 1024;     // slots per block of the histogram / scatter passes

// Device-side validation failures, numbered like PrefillMoEGroupingError's cases
// (PrefillMoEGrouping.swift:121-137).  The error word holds max over pairs of ~(index << 4 | code),
// i.e. the first failing pair in input order, as the reference's loop reports it; 0 = none.
// It lives in the context's persistent zeroed words and the scan kernel clears it again.
enum : uint32_t { GROUP_ERR_TOKEN = 6, GROUP_ERR_RANK = 7, GROUP_ERR_EXPERT = 8, GROUP_ERR_DUP = 9 };
constexpr uint32_t GROUP_UNCLAIMED = 0xFFFFFFFFu;

__global__ __launch_bounds__(256) void prefill_init_kernel(uint32_t* first, uint32_t n_pairs) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n_pairs) first[i] = GROUP_UNCLAIMED;
}

// PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:97-117): token-major records.
__global__ __launch_bounds__(256) void prefill_make_pairs_kernel(const uint32_t* idx, const uint16_t* w,
                                                                uint32_t n_pairs, uint32_t top_k,
                                                                PrefillPair* pairs) {
    const uint32_t p = blockIdx.x * 256 + threadIdx.x;
    if (p < n_pairs) pairs[p] = PrefillPair{p / top_k, idx[p], p % top_k, (uint32_t)w[p]};
}

// ---- pairs in any order -> slots (token * top_k + rank) ------------------------------------
// A valid input holds every slot exactly once, so sorting by (key, expert, token, rank) is a
// counting sort by expert over the slots in ascending order.
__global__ __launch_bounds__(256) void prefill_claim_kernel(const PrefillPair* pairs, uint32_t n_pairs,
                                                           uint32_t query_count, uint32_t top_k,
                                                           uint32_t num_experts, uint32_t* first,
                                                           uint32_t* words) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_pairs) return;
    const PrefillPair p = pairs[i];
    uint32_t code = 0;
    if (p.token >= query_count) code = GROUP_ERR_TOKEN;
    else if (p.rank >= top_k) code = GROUP_ERR_RANK;
    else if (p.expert >= num_experts) code = GROUP_ERR_EXPERT;
    if (code) atomicMax(&words[0], ~(i << 4 | code));
    else atomicMin(&first[p.token * top_k + p.rank], i);
}

__global__ __launch_bounds__(256) void prefill_slot_kernel(const PrefillPair* pairs, uint32_t n_pairs,
                                                          uint32_t query_count, uint32_t top_k,
                                                          uint32_t num_experts, const uint32_t* first,
                                                          uint32_t* slot_expert, uint32_t* slot_weight,
                                                          uint32_t* words) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_pairs) return;
    const PrefillPair p = pairs[i];
    if (p.token >= query_count || p.rank >= top_k || p.expert >= num_experts) return;
    const uint32_t slot = p.token * top_k + p.rank;
    if (first[slot] == i) { slot_expert[slot] = p.expert; slot_weight[slot] = p.weight_bits; }
    else atomicMax(&words[0], ~(i << 4 | GROUP_ERR_DUP));       // a later pair of an already seen slot
}

// ---- pass 1: per-block histogram of expert ids ------------------------------------------
// An unfilled slot (only after a validation error) may hold anything: ids out of range are
// skipped here and in the scatter, so every later index stays inside its array.  `report`:
// the ids come straight from a router and have not been range-checked yet.
__global__ __launch_bounds__(256) void prefill_hist_kernel(const uint32_t* idx, uint32_t n_pairs,
                                                          uint32_t num_experts, uint32_t* block_hist,
                                                          uint32_t* words, bool report) {
    extern __shared__ uint32_t lds[];
    for (uint32_t e = threadIdx.x; e < num_experts; e += 256) lds[e] = 0;
    __syncthreads();
    const uint32_t base = blockIdx.x * GROUP_CHUNK;
    for (uint32_t i = threadIdx.x; i < GROUP_CHUNK && base + i < n_pairs; i += 256) {
        const uint32_t e = idx[base + i];
        if (e < num_experts) atomicAdd(&lds[e], 1u);
        else if (report) atomicMax(&words[0], ~((base + i) << 4 | GROUP_ERR_EXPERT));
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < num_experts; e += 256) block_hist[(size_t)blockIdx.x * num_experts + e] = lds[e];
}

// ---- pass 2: offsets, counts, groups, tiles (PrefillMoEGrouping.swift:151-184) ------------
// Exclusive scan over the 1024 threads of the block; `total` is the sum over all of them.
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* wave_tot, uint32_t& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t t = (uint32_t)__shfl_up((int)inc, off, 64);
        if (lane >= off) inc += t;
    }
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    uint32_t before = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        const uint32_t t = wave_tot[w];
        before += w < wave ? t : 0u;
        tot += t;
    }
    __syncthreads();
    total = tot;
    return before + inc - v;
}

// One block.  Experts are laid out in ascending (sort key, expert) order; offsets of empty
// experts are 0xFFFFFFFF.  block_base[b][e] = first sorted slot of expert e's pairs of block b.
// info: [0] groups, [1] tiles, [2] error code (0 = none), [3] index of the failing pair,
// [4] largest group.  The error word is read and cleared for the next call.
__global__ __launch_bounds__(1024) void prefill_scan_kernel(const uint32_t* __restrict__ block_hist,
                                                           uint32_t* __restrict__ block_base, uint32_t n_blocks,
                                                           uint32_t num_experts, const uint64_t* sort_keys,
                                                           uint32_t tile_expert_count, uint32_t* offsets,
                                                           uint32_t* counts, PrefillGroup* groups,
                                                           PrefillTile* tiles, uint32_t* err_word, uint32_t* info) {
    extern __shared__ uint32_t lds[];
    uint32_t* cnt = lds;                       // [E] pairs of expert e
    uint32_t* order = lds + num_experts;       // [E] expert at position i of the key order
    uint32_t* start = lds + 2 * num_experts;   // [E] first pair of expert e
    uint32_t* gstart = lds + 3 * num_experts;  // [E] first pair of group g
    uint32_t* gcount = lds + 4 * num_experts;  // [E] pairs of group g
    uint32_t* misc = lds + 5 * num_experts;    // [0..15] wave totals, [16] largest group
    if (threadIdx.x == 0) misc[16] = 0;
    for (uint32_t e = threadIdx.x; e < num_experts; e += 1024) {
        uint32_t total = 0;
        for (uint32_t b = 0; b < n_blocks; ++b) total += block_hist[(size_t)b * num_experts + e];
        cnt[e] = total;
        uint32_t pos = e;
        if (sort_keys) {                                          // rank in (key, expert) order
            pos = 0;
            const uint64_t my_key = sort_keys[e];
            for (uint32_t o = 0; o < num_experts; ++o) {
                const uint64_t k = sort_keys[o];
                pos += (k < my_key || (k == my_key && o < e)) ? 1u : 0u;
            }
        }
        order[pos] = e;
    }
    __syncthreads();
    uint32_t pair_carry = 0, group_carry = 0;
    for (uint32_t base = 0; base < num_experts; base += 1024) {   // uniform trip count
        const uint32_t i = base + threadIdx.x;
        const uint32_t ex = i < num_experts ? order[i] : 0u;
        const uint32_t c = i < num_experts ? cnt[ex] : 0u;
        uint32_t pair_total, group_total;
        const uint32_t first = pair_carry + block_excl_scan(c, misc, pair_total);
        const uint32_t g = group_carry + block_excl_scan(c ? 1u : 0u, misc, group_total);
        if (i < num_experts) start[ex] = first;
        if (c) {
            groups[g] = PrefillGroup{ex, first, c};
            gstart[g] = first;
            gcount[g] = c;
            atomicMax(&misc[16], c);
        }
        pair_carry += pair_total;
        group_carry += group_total;
    }
    __syncthreads();
    const uint32_t ng = group_carry;
    const uint32_t nt = (ng + tile_expert_count - 1) / tile_expert_count;
    for (uint32_t t = threadIdx.x; t < nt; t += 1024) {
        const uint32_t gs = t * tile_expert_count, ge = min(ng, gs + tile_expert_count);
        tiles[t] = PrefillTile{gs, ge - gs, gstart[gs], gstart[ge - 1] + gcount[ge - 1] - gstart[gs]};
    }
    if (threadIdx.x == 0) {
        const uint32_t err = *err_word;            // 0 = none, else ~(index << 4 | code)
        *err_word = 0;
        info[0] = ng;
        info[1] = nt;
        info[2] = err ? (~err & 15u) : 0u;
        info[3] = err ? (~err >> 4) : 0u;
        info[4] = misc[16];
    }
    for (uint32_t e = threadIdx.x; e < num_experts; e += 1024) {
        counts[e] = cnt[e];
        offsets[e] = cnt[e] ? start[e] : 0xFFFFFFFFu;
        uint32_t run = start[e];
        for (uint32_t b0 = 0; b0 < n_blocks; b0 += 8) {
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) c[j] = b0 + j < n_blocks ? block_hist[(size_t)(b0 + j) * num_experts + e] : 0u;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (b0 + j < n_blocks) block_base[(size_t)(b0 + j) * num_experts + e] = run;
                run += c[j];
            }
        }
    }
}

// ---- pass 3: stable scatter ---------------------------------------------------------------
// Slots ascend in (token, rank).  A block places its slots 256 at a time; inside a round the
// four waves take turns, and inside a wave a lane's place among the lanes of the same expert
// comes from a ballot, so every expert keeps (token, rank) ascending: the order
// PrefillMoEGrouping.swift:140-149 sorts into.
__global__ __launch_bounds__(256) void prefill_scatter_kernel(const uint32_t* idx, const uint32_t* w32,
                                                             const uint16_t* w16, uint32_t n_pairs,
                                                             uint32_t top_k, uint32_t num_experts,
                                                             const uint32_t* block_base, PrefillPair* sorted) {
    extern __shared__ uint32_t next[];    // [E] next free sorted slot of each expert
    for (uint32_t e = threadIdx.x; e < num_experts; e += 256) next[e] = block_base[(size_t)blockIdx.x * num_experts + e];
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t base = blockIdx.x * GROUP_CHUNK;
    for (uint32_t r = 0; r < GROUP_CHUNK / 256; ++r) {          // uniform trip count: barriers inside
        const uint32_t p = base + r * 256 + threadIdx.x;
        uint32_t e = p < n_pairs ? idx[p] : 0xFFFFFFFFu;
        const bool valid = e < num_experts;
        const uint32_t wbits = valid ? (w32 ? w32[p] : (uint32_t)w16[p]) : 0u;
        uint32_t rank = 0, total = 0;
        bool leader = false;
        unsigned long long todo = __ballot(valid);
        while (todo) {                                           // one turn per distinct expert in the wave
            const int first = __builtin_ctzll(todo);
            const uint32_t le = (uint32_t)__builtin_amdgcn_readlane((int)e, first);
            const unsigned long long m = __ballot(valid && e == le);
            if (valid && e == le) {
                rank = (uint32_t)__builtin_popcountll(m & ((1ull << lane) - 1ull));
                total = (uint32_t)__builtin_popcountll(m);
                leader = lane == (uint32_t)first;
            }
            todo &= ~m;
        }
        for (uint32_t w = 0; w < 4; ++w) {
            if (wave == w && valid) {
                const uint32_t pos = next[e] + rank;             // every lane reads before the leader adds
                sorted[pos] = PrefillPair{p / top_k, e, p % top_k, wbits};
                if (leader) next[e] += total;
            }
            __syncthreads();
        }
    }
}

// ---- passes 2 and 3 in one launch, for inputs whose histogram is small -----------------------
// Every block repeats the scan over experts for itself (a few thousand additions), so nothing
// waits for a one-block launch in between: the block's first sorted slot of expert e is the
// expert's first slot plus the pairs of e in earlier blocks.  Block 0 also writes what the scan
// pass writes.  Inside a block wave w places slots [256 w, 256 w + 256) of the chunk, 64 at a
// time; a lane's place among the lanes of the same expert comes from one ballot per bit of the
// expert id, and per-wave counters carry it from one 64 to the next, so the four waves never
// wait for each other and every expert keeps (token, rank) ascending.
constexpr uint32_t FUSED_MAX_EXPERTS = 512, FUSED_MAX_BLOCKS = 64;

// Exclusive scan over the 256 threads of the block; `total` is the sum over all of them.
__device__ __forceinline__ uint32_t block256_excl_scan(uint32_t v, uint32_t* wave_tot, uint32_t& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t t = (uint32_t)__shfl_up((int)inc, off, 64);
        if (lane >= off) inc += t;
    }
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    uint32_t before = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t t = wave_tot[w];
        before += w < wave ? t : 0u;
        tot += t;
    }
    __syncthreads();
    total = tot;
    return before + inc - v;
}

__global__ __launch_bounds__(256) void prefill_scan_scatter_kernel(
    const uint32_t* __restrict__ idx, const uint32_t* __restrict__ w32, const uint16_t* __restrict__ w16,
    uint32_t n_pairs, uint32_t top_k, uint32_t num_experts, uint32_t id_bits,
    const uint32_t* __restrict__ block_hist, uint32_t n_blocks, const uint64_t* __restrict__ sort_keys,
    uint32_t tile_expert_count, uint32_t* offsets, uint32_t* counts, PrefillGroup* groups, PrefillTile* tiles,
    uint32_t* err_word, uint32_t* info, PrefillPair* sorted) {
    extern __shared__ uint32_t lds[];
    const uint32_t E = num_experts;
    uint32_t* cnt = lds;                 // [E] pairs of expert e
    uint32_t* before = lds + E;          // [E] of them in earlier blocks
    uint32_t* order = lds + 2 * E;       // [E] expert at position i of the key order
    uint32_t* start = lds + 3 * E;       // [E] first pair of expert e
    uint32_t* gstart = lds + 4 * E;      // [E] first pair of group g
    uint32_t* gcount = lds + 5 * E;      // [E] pairs of group g
    uint32_t* wnext = lds + 6 * E;       // [4][E] per wave: pairs of e, then next free slot of e
    uint32_t* misc = lds + 10 * E;       // [0..3] wave totals, [4] largest group
    uint64_t* keys = reinterpret_cast<uint64_t*>(lds + 10 * E + 8);   // [E]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) misc[4] = 0;
    for (uint32_t e = tid; e < E; e += 256) {
        uint32_t total = 0, earlier = 0;
        for (uint32_t b0 = 0; b0 < n_blocks; b0 += 8) {
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) c[j] = b0 + j < n_blocks ? block_hist[(size_t)(b0 + j) * E + e] : 0u;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                total += c[j];
                earlier += b0 + j < blockIdx.x ? c[j] : 0u;
            }
        }
        cnt[e] = total;
        before[e] = earlier;
        if (sort_keys) keys[e] = sort_keys[e];
#pragma unroll
        for (int w = 0; w < 4; ++w) wnext[w * E + e] = 0;
    }
    __syncthreads();
    for (uint32_t e = tid; e < E; e += 256) {
        uint32_t pos = e;
        if (sort_keys) {                                          // rank in (key, expert) order
            pos = 0;
            const uint64_t my_key = keys[e];
            for (uint32_t o = 0; o < E; ++o) {
                const uint64_t k = keys[o];
                pos += (k < my_key || (k == my_key && o < e)) ? 1u : 0u;
            }
        }
        order[pos] = e;
    }
    __syncthreads();
    uint32_t pair_carry = 0, group_carry = 0;
    for (uint32_t base = 0; base < E; base += 256) {              // uniform trip count
        const uint32_t i = base + tid;
        const uint32_t ex = i < E ? order[i] : 0u;
        const uint32_t c = i < E ? cnt[ex] : 0u;
        uint32_t pair_total, group_total;
        const uint32_t first = pair_carry + block256_excl_scan(c, misc, pair_total);
        const uint32_t g = group_carry + block256_excl_scan(c ? 1u : 0u, misc, group_total);
        if (i < E) start[ex] = first;
        if (c) {
            gstart[g] = first;
            gcount[g] = c;
            if (blockIdx.x == 0) {
                groups[g] = PrefillGroup{ex, first, c};
                atomicMax(&misc[4], c);
            }
        }
        pair_carry += pair_total;
        group_carry += group_total;
    }
    // ---- this block's slots: the lane's four, counted per wave
    const uint32_t base = blockIdx.x * GROUP_CHUNK + wave * 256 + lane;
    uint32_t ex[4], wbits[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t p = base + r * 64;
        ex[r] = p < n_pairs ? idx[p] : 0xFFFFFFFFu;
        wbits[r] = ex[r] < E ? (w32 ? w32[p] : (uint32_t)w16[p]) : 0u;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
        if (ex[r] < E) atomicAdd(&wnext[wave * E + ex[r]], 1u);
    __syncthreads();
    if (blockIdx.x == 0) {                                        // what the scan pass reports
        const uint32_t ng = group_carry;
        const uint32_t nt = (ng + tile_expert_count - 1) / tile_expert_count;
        for (uint32_t t = tid; t < nt; t += 256) {
            const uint32_t gs = t * tile_expert_count, ge = min(ng, gs + tile_expert_count);
            tiles[t] = PrefillTile{gs, ge - gs, gstart[gs], gstart[ge - 1] + gcount[ge - 1] - gstart[gs]};
        }
        if (tid == 0) {
            const uint32_t err = *err_word;        // 0 = none, else ~(index << 4 | code)
            *err_word = 0;
            info[0] = ng;
            info[1] = nt;
            info[2] = err ? (~err & 15u) : 0u;
            info[3] = err ? (~err >> 4) : 0u;
            info[4] = misc[4];
        }
        for (uint32_t e = tid; e < E; e += 256) {
            counts[e] = cnt[e];
            offsets[e] = cnt[e] ? start[e] : 0xFFFFFFFFu;
        }
    }
    for (uint32_t e = tid; e < E; e += 256) {
        uint32_t run = start[e] + before[e];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t c = wnext[w * E + e];
            wnext[w * E + e] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t e = ex[r];
        const bool valid = e < E;
        unsigned long long same = __ballot(valid);
        for (uint32_t i = 0; i < id_bits; ++i) {
            const bool bit = (e >> i) & 1u;
            const unsigned long long b = __ballot(valid && bit);
            same &= bit ? b : ~b;
        }
        if (valid) {
            const uint32_t rank = (uint32_t)__builtin_popcountll(same & ((1ull << lane) - 1ull));
            const uint32_t p = base + r * 64;
            const uint32_t pos = wnext[wave * E + e] + rank;       // every lane reads before the first one adds
            sorted[pos] = PrefillPair{p / top_k, e, p % top_k, wbits[r]};
            if (rank == 0) wnext[wave * E + e] += (uint32_t)__builtin_popcountll(same);
        }
    }
}

// ---- M tiles of the grouped GEMM ----------------------------------------------------------
struct MTile { uint32_t expert, row_start, rows; };
constexpr int GEMM_BM = 128;

constexpr uint32_t GEMM_SHORT_ROWS = 32;   // M tiles of at most this many rows take the kernel's short body

// Work lists of the grouped GEMM: one list of M tiles per XCD.
//
// An M tile (at most GEMM_BM sorted pairs of one expert) streams and dequantizes the codes of its
// expert's matrix; M tiles of one expert that run on one XCD at about the same time find those
// codes in that XCD's L2 instead of fetching them again.  The GEMM grid is dealt to the XCDs
// round-robin and XCD x works through list x in order, so the lists are made per expert: the
// groups are cut into items of at most cap = max(2, ceil(tiles / 64)) consecutive M tiles (an item
// never spans two experts; the cap keeps one very popular expert from unbalancing the lists), the
// items are sorted by cost, largest first, and dealt over the eight lists in serpentine order
// (0..7, 7..0, ...), which keeps the totals of a sorted sequence within one item of each other.
// Inside a list the most expensive items come first and the short tiles last.
// No list may be longer than list_max, what the GEMM grid covers; lists that would be, and
// groupings with more items than the tables below hold, are dealt tile by tile instead.
//
// list_len: [GEMM_XCDS] tiles in each list.  mtiles: list x at mtiles + x * list_cap.
constexpr uint32_t GEMM_XCDS = 8;
constexpr uint32_t MTILES_MAX_ITEMS = 1280;            // items that are sorted

__device__ __forceinline__ uint32_t mtile_cost(uint32_t rows) {   // in sixteenths of a full tile
    return rows > 64 ? 16u : rows > GEMM_SHORT_ROWS ? 11u : rows > 16 ? 8u : 7u;
}

// On a grouping that failed validation (info[2] != 0) no tile is listed, and this block zeroes the
// caller's route partials instead (slowly: it is the error path), so that the reduce after it
// returns zeros, never whatever the buffer held.
__global__ __launch_bounds__(256) void prefill_mtiles_kernel(const PrefillGroup* groups, const uint32_t* info,
                                                            MTile* mtiles, uint32_t list_cap, uint32_t list_max,
                                                            uint32_t* list_len, uint4* partials_on_error,
                                                            uint64_t partials_chunks) {
    __shared__ uint32_t it_group[MTILES_MAX_ITEMS], it_first[MTILES_MAX_ITEMS];
    __shared__ __attribute__((aligned(16))) uint32_t it_key[MTILES_MAX_ITEMS];   // all different: the item index is part of the key
    __shared__ uint32_t it_at[MTILES_MAX_ITEMS];        // M tiles of the item, then: list << 24 | offset in the list
    __shared__ uint32_t by_rank[MTILES_MAX_ITEMS];
    __shared__ uint32_t total_tiles, n_extra, too_long;
    const uint32_t tid = threadIdx.x;
    if (tid == 0) { total_tiles = 0; n_extra = 0; too_long = 0; }
    __syncthreads();
    const uint32_t ng = info[2] ? 0u : info[0];               // nothing runs on a grouping that failed
    if (info[2] && partials_on_error)
        for (uint64_t i = tid; i < partials_chunks; i += 256) partials_on_error[i] = uint4{0, 0, 0, 0};
    for (uint32_t g = tid; g < ng; g += 256) atomicAdd(&total_tiles, (groups[g].pair_count + GEMM_BM - 1) / GEMM_BM);
    __syncthreads();
    const uint32_t cap_tiles = max(2u, (total_tiles + 63u) / 64u);
    // tile by tile in group order: list lengths differ by at most one
    auto deal_tiles = [&]() {
        if (tid == 0) {
            uint32_t n = 0;
            for (uint32_t g = 0; g < ng; ++g) {
                const PrefillGroup gr = groups[g];
                for (uint32_t r = 0; r < gr.pair_count; r += GEMM_BM, ++n)
                    mtiles[(size_t)(n % GEMM_XCDS) * list_cap + n / GEMM_XCDS] =
                        MTile{gr.expert, gr.pair_start + r, gr.pair_count - r < (uint32_t)GEMM_BM ? gr.pair_count - r : (uint32_t)GEMM_BM};
            }
            for (uint32_t x = 0; x < GEMM_XCDS; ++x) list_len[x] = n / GEMM_XCDS + (x < n % GEMM_XCDS ? 1u : 0u);
        }
    };
    if (ng + 68u > MTILES_MAX_ITEMS) { deal_tiles(); return; }
    // items: the first of a group at the group's index, further ones behind the groups
    auto item_key = [&](const PrefillGroup& gr, uint32_t first, uint32_t item) {
        const uint32_t t = (gr.pair_count + GEMM_BM - 1) / GEMM_BM;
        const uint32_t n = min(cap_tiles, t - first);
        const uint32_t cost = (n - 1) * 16u + mtile_cost(first + n == t ? gr.pair_count - (t - 1) * GEMM_BM : (uint32_t)GEMM_BM);
        return (cost << 12) | (0xFFFu - (item & 0xFFFu));     // larger cost first, then lower index
    };
    for (uint32_t g = tid; g < ng; g += 256) {
        const PrefillGroup gr = groups[g];
        const uint32_t t = (gr.pair_count + GEMM_BM - 1) / GEMM_BM;
        it_group[g] = g; it_first[g] = 0; it_key[g] = item_key(gr, 0, g); it_at[g] = min(cap_tiles, t);
        for (uint32_t first = cap_tiles; first < t; first += cap_tiles) {
            const uint32_t i = ng + atomicAdd(&n_extra, 1u);  // at most 64 of them: total_tiles / cap_tiles
            it_group[i] = g; it_first[i] = first; it_key[i] = item_key(gr, first, i); it_at[i] = min(cap_tiles, t - first);
        }
    }
    __syncthreads();
    const uint32_t n_items = ng + n_extra;
    if (tid < 4 && n_items + tid < MTILES_MAX_ITEMS) it_key[n_items + tid] = 0;   // pads the last group of four
    __syncthreads();
    for (uint32_t i = tid; i < n_items; i += 256) {           // rank = keys above this one, four keys per read
        const uint32_t k = it_key[i];
        uint32_t r = 0;
        for (uint32_t j = 0; j < n_items; j += 4) {
            const uint4 o = *reinterpret_cast<const uint4*>(&it_key[j]);
            r += (o.x > k ? 1u : 0u) + (o.y > k ? 1u : 0u) + (o.z > k ? 1u : 0u) + (o.w > k ? 1u : 0u);
        }
        by_rank[r] = i;
    }
    __syncthreads();
    // serpentine deal: rank r -> row r / 8, list r % 8 on even rows, 7 - r % 8 on odd ones; one
    // thread per list walks its items in rank order and hands out the offsets (a chain of
    // dependent reads: everything it touches is in LDS)
    if (tid < GEMM_XCDS) {
        uint32_t at = 0;
        for (uint32_t row = 0; row * GEMM_XCDS < n_items; ++row) {
            const uint32_t r = row * GEMM_XCDS + ((row & 1u) ? GEMM_XCDS - 1u - tid : tid);
            if (r >= n_items) continue;
            const uint32_t i = by_rank[r];
            const uint32_t n = it_at[i];
            it_at[i] = (tid << 24) | at;
            at += n;
        }
        list_len[tid] = at;
        if (at > list_max) too_long = 1;
    }
    __syncthreads();
    if (too_long) { deal_tiles(); return; }                   // not reached for a sorted sequence; kept as the guarantee
    for (uint32_t i = tid; i < n_items; i += 256) {
        const PrefillGroup gr = groups[it_group[i]];
        const uint32_t t = (gr.pair_count + GEMM_BM - 1) / GEMM_BM;
        const uint32_t n = min(cap_tiles, t - it_first[i]);
        MTile* dst = mtiles + (size_t)(it_at[i] >> 24) * list_cap + (it_at[i] & 0xFFFFFFu);
        for (uint32_t j = 0; j < n; ++j) {
            const uint32_t r0 = (it_first[i] + j) * GEMM_BM;
            dst[j] = MTile{gr.expert, gr.pair_start + r0, min((uint32_t)GEMM_BM, gr.pair_count - r0)};
        }
    }
}

// ---- one streamed tile: experts bound one by one ----------------------------------------------
// The reference runs a tile of at most sixteen experts whose blobs were fetched into separate
// buffers (PrefillStreamedTileBinding, PrefillGroupedRoutedMoE.swift:185-323) over the sorted pairs
// [pair_start, pair_start + pair_count) (PrefillGroupedRoutedMoEStreamedParams, :104-183 ==
// prefill.metal:231-264).  This kernel turns such a call into the GEMM's work lists: the run of
// each bound expert inside the pair range (the pairs are sorted, so an expert's pairs are one
// run) is cut into M tiles whose `expert` is the LOCAL slot, dealt tile by tile over the lists,
// and the slots' blob addresses go into the table the GEMM reads.  A pair whose expert is not
// bound (validateCoversPairs, :274-287) lists nothing and reports (1, pair index) in err.
constexpr uint32_t STREAMED_MAX_EXPERTS = 16;
struct StreamedBind {
    const uint8_t* blob[STREAMED_MAX_EXPERTS];
    uint32_t expert[STREAMED_MAX_EXPERTS];      // global expert id of local slot i
    uint32_t live, pair_start, pair_count;
};

__global__ __launch_bounds__(256) void prefill_streamed_mtiles_kernel(const PrefillPair* pairs, StreamedBind b,
                                                                     const uint8_t** table, MTile* mtiles,
                                                                     uint32_t list_cap, uint32_t* list_len,
                                                                     uint32_t* err) {
    __shared__ uint32_t start[STREAMED_MAX_EXPERTS], stop[STREAMED_MAX_EXPERTS];
    __shared__ uint32_t bad;
    const uint32_t tid = threadIdx.x;
    if (tid < STREAMED_MAX_EXPERTS) {
        start[tid] = 0; stop[tid] = 0;
        table[tid] = tid < b.live ? b.blob[tid] : nullptr;
    }
    if (tid == 0) bad = 0xFFFFFFFFu;
    __syncthreads();
    const uint32_t lo = b.pair_start, hi = b.pair_start + b.pair_count;
    for (uint32_t i = lo + tid; i < hi; i += 256) {
        const uint32_t e = pairs[i].expert;
        const bool first = i == lo || pairs[i - 1].expert != e;
        const bool last = i + 1 == hi || pairs[i + 1].expert != e;
        if (!first && !last) continue;
        uint32_t slot = STREAMED_MAX_EXPERTS;
        for (uint32_t j = 0; j < b.live; ++j)
            if (b.expert[j] == e) { slot = j; break; }
        if (slot == STREAMED_MAX_EXPERTS) { atomicMin(&bad, i); continue; }
        if (first) start[slot] = i;
        if (last) stop[slot] = i + 1;
    }
    __syncthreads();
    if (tid != 0) return;
    if (err) { err[0] = bad != 0xFFFFFFFFu ? 1u : 0u; err[1] = bad != 0xFFFFFFFFu ? bad : 0u; }
    uint32_t n = 0;
    if (bad == 0xFFFFFFFFu) {
        for (uint32_t slot = 0; slot < b.live; ++slot)
            for (uint32_t r = start[slot]; r < stop[slot]; r += GEMM_BM, ++n)
                mtiles[(size_t)(n % GEMM_XCDS) * list_cap + n / GEMM_XCDS] =
                    MTile{slot, r, stop[slot] - r < (uint32_t)GEMM_BM ? stop[slot] - r : (uint32_t)GEMM_BM};
    }
    for (uint32_t x = 0; x < GEMM_XCDS; ++x) list_len[x] = n / GEMM_XCDS + (x < n % GEMM_XCDS ? 1u : 0u);
}

// ---- grouped GEMM ---------------------------------------------------------------------------
// out[m, n] = sum_k X[row(m), k] * W_e[n, k] for the rows of one M tile (<= 128 sorted pairs of
// one expert) and GEMM_BN output columns: DUAL -> gate and up rows of the same columns,
// epilogue silu(g) * u (prefill.metal:460-501); else down rows (prefill.metal:503-534).
//
// k runs in super-steps of 128 (two quantization groups).  The activations of a super-step sit
// in an LDS stage shared by the four waves.  Wave w owns 16 * NT columns of all 128 rows, and
// lane (i = lane % 16, q = lane / 16) holds the 32 codes W[n_i, k0 + 32q .. +32) of each of its
// columns, fetched in one 16-byte (4 bit) or two (8 bit) loads, so four neighbouring lanes
// cover 64 or 128 contiguous bytes of a row.  It dequantizes them in registers,
// w = q * scale + bias in fp32 rounded once to the activation type (the reference dequantizes
// to fp16, tensorops.metal:29-121), straight into the MFMA B operand: MFMA j of the super-step
// contracts k0 + 32q + 8j .. +8 over q = 0..3, and the A operand is read from LDS with the same
// k assignment.  v_mfma_f32_16x16x32_{bf16,f16} accumulates in fp32.
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
typedef _Float16 hf8_t __attribute__((ext_vector_type(8)));
typedef _Float16 hf2_t __attribute__((ext_vector_type(2)));
typedef float fl2_t __attribute__((ext_vector_type(2)));
typedef float fl4_t __attribute__((ext_vector_type(4)));

struct GemmParams {
    const uint8_t* pool;
    uint64_t pool_stride;
    const uint8_t* const* blob_table;   // optional: expert e's blob at blob_table[e] (experts bound one by one,
                                        // PrefillStreamedTileBinding) instead of pool + e * pool_stride
    int64_t wA, sA, bA, wB, sB, bB;     // A: gate or down; B: up
    const MTile* mtiles;                // grouped product: list x of M tiles at mtiles + x * list_cap
    uint32_t list_cap;
    const uint32_t* list_len;           // [GEMM_XCDS] tiles in each list
    const PrefillPair* pairs;           // sorted
    const void* x;                      // DUAL: hidden rows by token; else act rows by sorted position
    uint32_t x_stride;
    void* out;                          // DUAL: act[sorted position, N]; else partials[token*top_k+rank, N]
    uint32_t out_stride;
    uint32_t K, N, top_k, n_tiles_n;
    uint32_t dense_bm;                  // rows per M tile of a dense product: GEMM_BM, or 64 when the launch would
                                        // otherwise leave half of the block slots empty (dense_bm_for)
    uint32_t dense_rows;                // > 0: a dense product over rows 0..dense_rows-1 of x (row i -> row i of
                                        // out; DUAL: gate/up + SwiGLU of one expert over all rows), M tiles of
                                        // GEMM_BM consecutive rows; mtiles, n_mtiles, pairs unused
};

constexpr int GEMM_SK = 128;            // k per super-step
constexpr uint32_t GEMM_DENSE_MGROUP = 4; // M tiles of a dense product that an XCD sweeps the columns with

// Two floats -> two 16-bit activations in one dword, round to nearest even.
template <int ACT>
__device__ __forceinline__ uint32_t pack_act2(float lo, float hi) {
    const fl2_t v = {lo, hi};
    if (ACT == ACT_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2_t));   // v_cvt_pk_bf16_f32
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hf2_t));
}

template <int ACT>
__device__ __forceinline__ fl4_t mfma_16x16x32(const uint4& a, const uint4& b, fl4_t c) {
    if (ACT == ACT_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, a), __builtin_bit_cast(bf8_t, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(hf8_t, a), __builtin_bit_cast(hf8_t, b), c, 0, 0, 0);
}

// Eight codes -> eight dequantized 16-bit values in MFMA operand order.
template <int ACT>
__device__ __forceinline__ uint4 dequant8(const float* q, float s, float b) {
    uint4 o;
    o.x = pack_act2<ACT>(fmaf(q[0], s, b), fmaf(q[1], s, b));
    o.y = pack_act2<ACT>(fmaf(q[2], s, b), fmaf(q[3], s, b));
    o.z = pack_act2<ACT>(fmaf(q[4], s, b), fmaf(q[5], s, b));
    o.w = pack_act2<ACT>(fmaf(q[6], s, b), fmaf(q[7], s, b));
    return o;
}

// Eight codes of one dword (4 bit) or of two (8 bit) -> eight dequantized 16-bit values in MFMA
// operand order, through fp16 "magic" pairs: (code | 0x6400) is the fp16 number 1024 + code, two
// of them are made by one AND-OR, and the mixed-precision FMA reads either half directly, so
// no code is converted to float on its own: w = (1024 + q) * s + (b - 1024 s).  The shifted bias
// is rounded once in fp32 (error below 2^-14 of a quantization step).  mask (0x000F000F or
// 0x00FF00FF) and magic (0x64006400) arrive in registers: as literals they would split every
// AND-OR in two, a three-operand instruction takes no literal here.
// Measured and not kept: the result written as fp16 halves by v_fma_mixlo_f16 / v_fma_mixhi_f16
// (no pack instructions, but the two issue at half the rate of v_fma_mix_f32: 18 % fewer vector
// instructions, 7 % more vector cycles, 5 % slower); 4-bit pairs without two of the three shifts
// (a nibble at bits 4..7 of a half as 64 + q under 0x5400, with a second shifted bias): four
// more registers live across the loop, which the 256-register kernels do not have (52 bytes of
// scratch, 8 % slower); 8-bit pairs by one byte permute each instead of shift + AND-OR (equal).
template <int ACT, int BITS>
__device__ __forceinline__ uint4 dequant8_magic(uint32_t w0, uint32_t w1, float s, float b1024, uint32_t mask, uint32_t magic) {
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    uint32_t pr[4];                         // pr[i] = (code lo_i, code hi_i) as fp16 pairs
    int lo_of[8], half_of[8];               // element e sits in pr[lo_of[e]], half half_of[e]
    if (BITS == 4) {
        // dword w0: codes at bits 4e; pair i = (code i, code i + 4)
#pragma unroll
        for (int i = 0; i < 4; ++i) pr[i] = ((w0 >> (4 * i)) & mask) | magic;
#pragma unroll
        for (int e = 0; e < 8; ++e) { lo_of[e] = e & 3; half_of[e] = e >> 2; }
    } else {
        // bytes of w0 = codes 0..3, of w1 = codes 4..7; pair (0, 2), (1, 3) of each dword
        pr[0] = (w0 & mask) | magic;
        pr[1] = ((w0 >> 8) & mask) | magic;
        pr[2] = (w1 & mask) | magic;
        pr[3] = ((w1 >> 8) & mask) | magic;
#pragma unroll
        for (int e = 0; e < 8; ++e) { lo_of[e] = (e >> 2) * 2 + (e & 1); half_of[e] = (e >> 1) & 1; }
    }
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const h2_t h = __builtin_bit_cast(h2_t, pr[lo_of[e]]);
        v[e] = __builtin_fmaf((float)(half_of[e] ? h.y : h.x), s, b1024);
    }
    uint4 o;
    o.x = pack_act2<ACT>(v[0], v[1]);
    o.y = pack_act2<ACT>(v[2], v[3]);
    o.z = pack_act2<ACT>(v[4], v[5]);
    o.w = pack_act2<ACT>(v[6], v[7]);
    return o;
}

// NT = 16-column tiles per wave (2 or 4): the block covers 32 NT gate/up columns (DUAL) or
// 64 NT down columns.  NT = 4 reads each activation fragment from LDS once for four MFMAs and
// halves the number of blocks that re-read an M tile's activations.
//
// Activations reach LDS without passing through registers (buffer_load ... lds, 16 bytes per
// lane), the weights of the next super-step likewise.  Weight and scale loads are buffer loads:
// one lane offset each, the tile / matrix / super-step part in a scalar, so the loop carries two
// address registers for the weights instead of twenty-four.
//
// LDS of a block: two activation stages and 4 KB of weight stage per wave, 80 KB, so that two
// blocks share a compute unit's 160 KB.  They are three separate arrays on purpose: the
// compiler makes every LDS read wait for all LDS-bound loads in flight unless it can prove
// that they touch different memory, and it can for different arrays.  With one buffer the
// loads of the next stage would be waited for before the first fragment read of this one.
constexpr uint32_t GEMM_XBUF = GEMM_BM * GEMM_SK * 2;      // bytes of one activation stage

// Position swizzle of row r (0..15) of a 16-row tile whose rows are 64 bytes apart: the sixteen
// 16-byte reads of a fragment (one per row, same chunk) fall into sixteen different 16-byte
// bank groups of a 256-byte LDS line, and each half of them (rows 0..7, 8..15) into eight
// different groups of a 128-byte line.
__device__ __forceinline__ uint32_t gemm_row_swizzle(uint32_t r) { return ((r >> 1) & 3u) ^ (r >> 3); }

// s_waitcnt operand: at most n vector-memory loads still in flight, the other counters free.
constexpr int gemm_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

template <int ACT, int BITS, bool DUAL, int NT>
__global__ __launch_bounds__(256, 2) void prefill_gemm_kernel(GemmParams p) {
    constexpr int WQ = BITS == 8 ? 2 : 1;               // 16-byte loads per (column, super-step)
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint8_t xs0[GEMM_XBUF];
    __shared__ __attribute__((aligned(16))) uint8_t xs1[GEMM_XBUF];
    __shared__ __attribute__((aligned(16))) uint8_t ws[4 * 4096];
    // Arrays that only load instructions write look never-written to the optimizer, which would
    // then fold every read of them away: a store that never executes keeps them alive (the
    // entry points reject K = 0).
    if (p.K == 0) { xs1[threadIdx.x] = 0; ws[threadIdx.x] = 0; }
    // Blocks are dealt to the eight XCDs round-robin: block b runs on XCD b % 8, and an XCD takes
    // its blocks in the order of their indices.
    // Dense product: what an XCD's 128 resident blocks read should fit its L2.  With eight M tiles or more, XCD x
    // owns the M tiles x, x + 8, ... and takes them four at a time: for each column tile the four blocks of the
    // group, so the 128 blocks in flight are 32 column tiles against four M tiles -- 2 MB of activation rows stay
    // in the L2 while the codes stream through, each column tile fetched once for the four.  (Units of four column
    // tiles of one M tile dealt over the XCDs in turn, the order before this one, had some twenty M tiles and all
    // column groups in flight per XCD: 1,536 blocks of 800 KB each came from beyond the L2, 1.2 GB for a product
    // whose operands are 31 MB.  The time is the same, 241 against 245 us for 4096 x 12,352 x 2048: the memory
    // side cache absorbed it; what is saved is fabric traffic.)  With fewer M tiles, XCD x owns the column tiles
    // x, x + 8, ... instead and takes every M tile against each: the codes of a column tile are fetched into one
    // L2 only.
    // Grouped product: XCD x works through list x of the M tiles, every column tile of an M tile in
    // turn.  The column tiles of an M tile share its activation rows and the M tiles of an expert
    // (neighbours in a list) share its codes: both meet in that XCD's L2.
    const uint32_t on_xcd = blockIdx.x >> 3;
    MTile mt;
    uint32_t nt;
    if (p.dense_rows) {
        const uint32_t xcd = blockIdx.x & 7u, tiles_m = (p.dense_rows + p.dense_bm - 1) / p.dense_bm;
        uint32_t tile_id;
        if (tiles_m >= 8) {
            const uint32_t mine = (tiles_m - xcd + 7) / 8;                      // M tiles of this XCD
            const uint32_t full = mine / GEMM_DENSE_MGROUP * GEMM_DENSE_MGROUP;  // ... in whole groups
            uint32_t at;                                                         // which of them
            if (on_xcd < full * p.n_tiles_n) {
                const uint32_t grp = on_xcd / (GEMM_DENSE_MGROUP * p.n_tiles_n), in = on_xcd % (GEMM_DENSE_MGROUP * p.n_tiles_n);
                nt = in / GEMM_DENSE_MGROUP;
                at = grp * GEMM_DENSE_MGROUP + in % GEMM_DENSE_MGROUP;
            } else {
                const uint32_t rest = mine - full, in = on_xcd - full * p.n_tiles_n;
                if (rest == 0) return;
                nt = in / rest;
                at = full + in % rest;
            }
            tile_id = xcd + 8 * at;
        } else {
            nt = xcd + 8 * (on_xcd / tiles_m);
            tile_id = on_xcd % tiles_m;
        }
        if (tile_id * p.dense_bm >= p.dense_rows || nt >= p.n_tiles_n) return;
        mt = MTile{0u, tile_id * p.dense_bm, min(p.dense_bm, p.dense_rows - tile_id * p.dense_bm)};
    } else {
        const uint32_t list = blockIdx.x & (GEMM_XCDS - 1u), at = on_xcd / p.n_tiles_n;
        nt = on_xcd % p.n_tiles_n;
        if (at >= p.list_len[list]) return;
        mt = p.mtiles[(size_t)list * p.list_cap + at];
    }
    const uint8_t* blob = p.blob_table ? p.blob_table[mt.expert] : p.pool + (uint64_t)mt.expert * p.pool_stride;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const uint32_t groups = p.K / NVMAI_GROUP;
    constexpr uint32_t n_cols = DUAL ? 32 * NT : 64 * NT;   // output columns per block
    const uint32_t n0 = nt * n_cols;
    const int live_mt = (int)((mt.rows + 15) >> 4);     // 16-row tiles that hold any row
    const uint32_t nss = (p.K + GEMM_SK - 1) / GEMM_SK;
    // A K that is an odd multiple of 64 leaves half of the last super-step empty: lanes whose k
    // range lies beyond K contribute zeros (zero activations, zero weights).
    const bool odd_tail = (p.K % GEMM_SK) != 0;

    // ---- activations.  A stage holds 128 rows x 128 k as eight 4 KB blocks, one per 16-row
    // tile: [k quarter: 4][row: 16][position: 4] 16-byte chunks, chunk c of row r in quarter
    // c / 4 at position (c % 4) ^ swizzle(r).  An MFMA fragment read (16 rows, one chunk each) then
    // touches every bank once, and a load instruction (64 lanes x 16 bytes = one quarter of one
    // tile) needs only a lane-constant offset: wave w fills tiles 2 w and 2 w + 1, lane l row
    // l / 4 of the tile, so two address registers serve all eight loads of a super-step.
    // Tiles past the end of a short M tile are not loaded: their LDS rows keep whatever they
    // held, which only reaches accumulator rows that are never stored.
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(p.x), 0, (int)0xFFFFFFFFu, 0x00020000);
    uint32_t xoff[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        const uint32_t row = (wave * 2 + g) * 16 + (lane >> 2);
        const uint32_t m = row < mt.rows ? row : 0;     // a dead row of a live tile repeats row 0
        const uint32_t src = (DUAL && !p.dense_rows) ? p.pairs[mt.row_start + m].token : mt.row_start + m;
        xoff[g] = src * (p.x_stride * 2u) + (uint32_t)((lane & 3) ^ gemm_row_swizzle(lane >> 2)) * 16u;
    }
    auto load_x = [&](uint32_t ss, uint8_t* stage) {
        if (!(odd_tail && ss == nss - 1)) {
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                if ((wave * 2 + g) * 16 >= mt.rows) break;  // wave-uniform
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (__attribute__((address_space(3))) void*)(stage + (wave * 2 + g) * 4096 + i * 1024),
                                                             16, xoff[g], ss * (GEMM_SK * 2) + i * 64, 0, 0);
            }
        } else {
            // the last super-step of an odd K: its second half takes zeros, not loads
#pragma unroll 1
            for (int g = 0; g < 2; ++g) {
                if ((wave * 2 + g) * 16 >= mt.rows) break;
                uint8_t* dst = stage + (wave * 2 + g) * 4096;
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, xoff[g],
                                                             ss * (GEMM_SK * 2) + i * 64, 0, 0);
                *reinterpret_cast<uint4*>(dst + 2048 + lane * 16) = uint4{0, 0, 0, 0};
                *reinterpret_cast<uint4*>(dst + 3072 + lane * 16) = uint4{0, 0, 0, 0};
            }
        }
    };

    // ---- weight columns of this lane: tile t -> DUAL {gate, up}[t & 1] of column
    //      n0 + 8 NT wave + 16 (t / 2) + i, else column n0 + 16 NT wave + 16 t + i.
    // Columns past N (a last block that sticks out) read zeros; they are never stored.
    // One resource per array (codes, scales, biases of matrix A and, DUAL, of matrix B), bounded
    // by the array's size: the arrays of a dense product need not lie in one allocation.
    const uint32_t row_bytes = p.K * BITS / 8;
    const uint32_t w_bytes = p.N * row_bytes, sb_bytes = p.N * groups * 2u;
    auto rsrc_of = [&](int64_t off, uint32_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(blob + off), 0, (int)bytes, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t wrsA = rsrc_of(p.wA, w_bytes), wrsB = rsrc_of(DUAL ? p.wB : p.wA, w_bytes);
    const uint32_t col0 = DUAL ? n0 + wave * (8 * NT) + li : n0 + wave * (16 * NT) + li;
    const uint32_t wv = col0 * row_bytes + lq * (32 * BITS / 8);
    uint32_t wso[NT];                                   // scalar part: the tile's first column
#pragma unroll
    for (int t = 0; t < NT; ++t) wso[t] = (DUAL ? (t >> 1) * 16 : t * 16) * row_bytes;

    // ---- scales and biases.  A lane needs, per super-step and tile, the scale and bias of its
    // column for the group its k range lies in.  Loaded lane by lane those are 2 NT two-byte
    // loads per super-step whose 64 lanes hit 64 different cache lines each, and the address
    // path, not the matrix pipe, sets the pace of the kernel.  Instead lane 16 t + c fetches for
    // tile t, column c, the scales (and the biases) of CS super-steps at once: one wide load per
    // array per CS super-steps.  A consumer lane takes its dword (two groups) from the fetching
    // lane through the cross-lane network and keeps the half of its group.
    // Rows of scales start on 2-byte boundaries when K / 64 is odd: the load starts at the dword
    // below and takes one more, and a funnel shift lines the pairs up.
    const int ld_t = lane >> 4;
    const bool ld_on = NT == 4 || ld_t < NT;
    const bool ld_second = DUAL && (ld_t & 1);
    uint32_t so_lane, bo_lane;
    {
        uint32_t c = DUAL ? n0 + wave * (8 * NT) + (ld_t >> 1) * 16 + li : n0 + wave * (16 * NT) + ld_t * 16 + li;
        c = min(c, p.N - 1) * groups * 2u;
        so_lane = (DUAL ? (uint32_t)(ld_second ? p.sB : p.sA) : 0u) + c;
        bo_lane = (DUAL ? (uint32_t)(ld_second ? p.bB : p.bA) : 0u) + c;
    }
    // DUAL: gate and up arrays are reached from the expert's base (the lane picks the matrix)
    const uint32_t blob_bytes = (uint32_t)(p.pool_stride < 0xFFFFFFFFull ? p.pool_stride : 0xFFFFFFFFull);
    const __amdgpu_buffer_rsrc_t s_rs = DUAL ? rsrc_of(0, blob_bytes) : rsrc_of(p.sA, sb_bytes);
    const __amdgpu_buffer_rsrc_t b_rs = DUAL ? rsrc_of(0, blob_bytes) : rsrc_of(p.bA, sb_bytes);
    // raw: CS + 1 dwords from the dword at or below the row's chunk
    auto load_sb = [&](auto csc, uint32_t* rs_, uint32_t* rb_, uint32_t chunk) {
        constexpr int CS = decltype(csc)::value;
        if (ld_on) {
            if (CS == 1) {
                typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
                const u32x2_t a = __builtin_amdgcn_raw_buffer_load_b64(s_rs, so_lane & ~3u, chunk * 4, 0);
                const u32x2_t c = __builtin_amdgcn_raw_buffer_load_b64(b_rs, bo_lane & ~3u, chunk * 4, 0);
                rs_[0] = a.x; rs_[1] = a.y;
                rb_[0] = c.x; rb_[1] = c.y;
            } else if (CS == 2) {
                typedef uint32_t u32x3_t __attribute__((ext_vector_type(3)));
                const u32x3_t a = __builtin_amdgcn_raw_buffer_load_b96(s_rs, so_lane & ~3u, chunk * (CS * 4), 0);
                const u32x3_t c = __builtin_amdgcn_raw_buffer_load_b96(b_rs, bo_lane & ~3u, chunk * (CS * 4), 0);
                rs_[0] = a.x; rs_[1] = a.y; rs_[2] = a.z;
                rb_[0] = c.x; rb_[1] = c.y; rb_[2] = c.z;
            } else {
                const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(s_rs, so_lane & ~3u, chunk * (CS * 4), 0);
                const u32x4_t c = __builtin_amdgcn_raw_buffer_load_b128(b_rs, bo_lane & ~3u, chunk * (CS * 4), 0);
                rs_[0] = a.x; rs_[1] = a.y; rs_[2] = a.z; rs_[3] = a.w;
                rb_[0] = c.x; rb_[1] = c.y; rb_[2] = c.z; rb_[3] = c.w;
            }
        }
    };
    // raw -> CS dwords, one per super-step of the chunk: (scale of group 2 ss, of group 2 ss + 1)
    auto align_sb = [&](auto csc, const uint32_t* rs_, const uint32_t* rb_, uint32_t* cs_, uint32_t* cb_) {
        constexpr int CS = decltype(csc)::value;
#pragma unroll
        for (int h = 0; h < CS; ++h) {
            cs_[h] = __builtin_amdgcn_alignbit(rs_[h + 1], rs_[h], (so_lane & 2u) * 8u);
            cb_[h] = __builtin_amdgcn_alignbit(rb_[h + 1], rb_[h], (bo_lane & 2u) * 8u);
        }
    };
    // the fetching lanes' dwords of one super-step -> this lane's (scale, bias) per tile, packed:
    // scale in the high half, bias in the low half.  The cross-lane reads carry the tile in their
    // immediate offset, so one address register serves all of them.
    [[maybe_unused]] const uint32_t bp_addr = 4u * li;
    auto scales_from = [&](uint32_t s_dw, uint32_t b_dw, uint32_t ss, uint32_t* sb) {
        const bool dead = odd_tail && ss == nss - 1 && lq >= 2;
        uint32_t ds[4], db[4];
#if defined(__HIP_DEVICE_COMPILE__)
        if (NT == 4)
            asm volatile("ds_bpermute_b32 %0, %8, %9\n\tds_bpermute_b32 %1, %8, %9 offset:64\n\t"
                         "ds_bpermute_b32 %2, %8, %9 offset:128\n\tds_bpermute_b32 %3, %8, %9 offset:192\n\t"
                         "ds_bpermute_b32 %4, %8, %10\n\tds_bpermute_b32 %5, %8, %10 offset:64\n\t"
                         "ds_bpermute_b32 %6, %8, %10 offset:128\n\tds_bpermute_b32 %7, %8, %10 offset:192\n\t"
                         "s_waitcnt lgkmcnt(0)"
                         : "=&v"(ds[0]), "=&v"(ds[1]), "=&v"(ds[2]), "=&v"(ds[3]), "=&v"(db[0]), "=&v"(db[1]), "=&v"(db[2]), "=&v"(db[3])
                         : "v"(bp_addr), "v"(s_dw), "v"(b_dw));
        else
            asm volatile("ds_bpermute_b32 %0, %4, %5\n\tds_bpermute_b32 %1, %4, %5 offset:64\n\t"
                         "ds_bpermute_b32 %2, %4, %6\n\tds_bpermute_b32 %3, %4, %6 offset:64\n\t"
                         "s_waitcnt lgkmcnt(0)"
                         : "=&v"(ds[0]), "=&v"(ds[1]), "=&v"(db[0]), "=&v"(db[1])
                         : "v"(bp_addr), "v"(s_dw), "v"(b_dw));
#endif
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            // the group of this lane's k range is the low (lq < 2) or the high half of each dword
            const uint32_t pk = (lq >> 1) ? __builtin_amdgcn_perm(ds[t], db[t], 0x07060302u)
                                          : __builtin_amdgcn_perm(ds[t], db[t], 0x05040100u);
            sb[t] = dead ? 0u : pk;
        }
    };

    // The weights of the next super-step wait in a wave-private LDS stage (the lane's own 16
    // bytes per tile, written by the load itself), so that only the super-step being multiplied
    // occupies registers.
    uint8_t* wlds = ws + wave * (NT * WQ * 1024);
    uint4 wcur[NT][WQ];
    auto issue_w = [&](uint32_t ss) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const uint32_t so = wso[t] + ss * (GEMM_SK * BITS / 8);
#pragma unroll
            for (int h = 0; h < WQ; ++h)
                __builtin_amdgcn_raw_ptr_buffer_load_lds((DUAL && (t & 1)) ? wrsB : wrsA, (__attribute__((address_space(3))) void*)(wlds + (t * WQ + h) * 1024),
                                                         16, wv + 16 * h, so, 0, 0);
        }
    };
    // After vmcnt(0): the stage moves into registers.
    auto take_w = [&]() {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int h = 0; h < WQ; ++h)
                wcur[t][h] = *reinterpret_cast<const uint4*>(wlds + (t * WQ + h) * 1024 + lane * 16);
    };

    // The main loop is a flat pipeline over MFMA steps (four per super-step): while the matrix
    // pipe works through step s, the vector pipe dequantizes the operand of step s + 1 into the
    // other half of bf[], across super-step boundaries too.  MT = 16-row tiles multiplied
    // (1, 2, 4 or 8, block-uniform): the body holds no branch, so that the LDS reads of the next
    // row tile and the dequantization interleave with the MFMAs.
    uint32_t dq_mask = BITS == 4 ? 0x000F000Fu : 0x00FF00FFu, dq_magic = 0x64006400u;
#if defined(__HIP_DEVICE_COMPILE__)
    asm("" : "+s"(dq_mask));                            // opaque: kept in a scalar / a vector register
    asm("" : "+v"(dq_magic));
#endif
    auto dequant_step = [&](const uint4 (*w4)[WQ], const uint32_t* sb, int j, uint4* bfrag) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float sc = __builtin_bit_cast(float, sb[t] & 0xFFFF0000u);
            const float b1024 = __builtin_fmaf(-1024.0f, sc, __builtin_bit_cast(float, sb[t] << 16));
            if (BITS == 4) {
                const uint4 w = w4[t][0];
                bfrag[t] = dequant8_magic<ACT, 4>(j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w, 0u, sc, b1024, dq_mask, dq_magic);
            } else {
                const uint4 w = w4[t][j >> 1];
                bfrag[t] = dequant8_magic<ACT, 8>((j & 1) ? w.z : w.x, (j & 1) ? w.w : w.y, sc, b1024, dq_mask, dq_magic);
            }
        }
    };
    // LDS byte address of the lane's fragment of row tile 0, MFMA step 0, stage 0; step j: ^ 16 j
    const uint32_t xa0 = lq * 1024 + li * 64 + gemm_row_swizzle(li) * 16;
    // MFMAs of step j over MT row tiles of stage `cur`, and the issue order of the step: fragment
    // reads one row tile ahead of their MFMAs, the next operand's dequantization (already in the
    // instruction stream) spread between the MFMAs.  An MFMA occupies the matrix pipe for four
    // issue slots: three vector instructions of the same wave fit behind each one.
    auto mfma_step = [&](auto mtc, fl4_t (*acc)[NT], const uint8_t* cur, int j, const uint4* bfrag) {
        constexpr int MT = decltype(mtc)::value;
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            const uint4 afrag = *reinterpret_cast<const uint4*>(cur + (xa0 ^ (16u * j)) + a * 4096);
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[a][t] = mfma_16x16x32<ACT>(afrag, bfrag[t], acc[a][t]);
        }
        constexpr int VPER = ((BITS == 4 ? 23 : 21) + MT - 1) / MT;    // per MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, MT > 1 ? 2 : 1, 0);
#pragma unroll
        for (int a = 0; a < MT; ++a) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, VPER, 0);
            }
            if (a + 2 < MT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    // ---- epilogue: lane holds column i of each tile, rows 16 a + 4 q .. +4.  The output tile
    // is rounded to 16 bits into the first activation stage (free after the last barrier), AP
    // row tiles at a time, and leaves in 16-byte pieces, whole rows of the tile at a time.
    auto epilogue = [&](auto mtc, fl4_t (*acc)[NT]) {
        constexpr int MT = decltype(mtc)::value;
        constexpr int OC = n_cols;                          // columns of the block's tile
        constexpr int LDO = OC + 8;
        constexpr int AP0 = OC >= 256 ? 2 : OC >= 128 ? 4 : 8;  // 16 AP rows of LDO elements fit in 32 KB
        constexpr int AP = AP0 < MT ? AP0 : MT;
        static_assert(16 * AP * LDO * 2 <= (int)GEMM_XBUF, "epilogue tile exceeds an activation stage");
        uint16_t* os = reinterpret_cast<uint16_t*>(xs0);
        constexpr int PIECES = OC / 8;                      // 16-byte pieces per row
        constexpr int ROWS_PER_PASS = 256 / PIECES;
        const int piece = tid % PIECES, prow = tid / PIECES;
        uint16_t* out = (uint16_t*)p.out;
        const bool vec_ok = (p.out_stride % 8 == 0) && n0 + OC <= p.N;
        // Down projection: a row's destination comes from its pair record.  All of them are
        // fetched now, in one round trip, into the second activation stage; fetched row by row
        // inside the store loop each one would be a dependent global load.
        uint32_t* orow_tab = reinterpret_cast<uint32_t*>(xs1);
        if (!DUAL && (uint32_t)tid < mt.rows) {
            if (p.dense_rows) orow_tab[tid] = mt.row_start + tid;
            else {
                const PrefillPair pr = p.pairs[mt.row_start + tid];
                orow_tab[tid] = pr.token * p.top_k + pr.rank;
            }
        }
#pragma unroll
        for (int a0 = 0; a0 < MT; a0 += AP) {
            if (a0 >= live_mt) break;                       // block-uniform
#pragma unroll
            for (int da = 0; da < AP; ++da) {
                const int a = a0 + da;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = da * 16 + lq * 4 + r;
                    if (DUAL) {
#pragma unroll
                        for (int c = 0; c < NT / 2; ++c)
                            os[m * LDO + wave * (8 * NT) + c * 16 + li] =
                                f32_to_act<ACT>(silu_fast(acc[a][2 * c][r]) * acc[a][2 * c + 1][r]);
                    } else {
#pragma unroll
                        for (int t = 0; t < NT; ++t) os[m * LDO + wave * (16 * NT) + t * 16 + li] = f32_to_act<ACT>(acc[a][t][r]);
                    }
                }
            }
            __syncthreads();
            const uint32_t m_end = min(mt.rows, (uint32_t)(a0 + AP) * 16u);
            for (uint32_t m = a0 * 16 + prow; m < m_end; m += ROWS_PER_PASS) {
                const size_t orow = (size_t)(DUAL ? mt.row_start + m : orow_tab[m]) * p.out_stride;
                const uint4 v = *reinterpret_cast<const uint4*>(os + (m - a0 * 16) * LDO + piece * 8);
                const uint32_t c0 = n0 + piece * 8;
                if (vec_ok) *reinterpret_cast<uint4*>(out + orow + c0) = v;
                else {
                    const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (c0 + j < p.N) out[orow + c0 + j] = e[j];
                }
            }
            if (a0 + AP < MT) __syncthreads();
        }
    };

    // ---- 3 to 8 row tiles (MT = 4 or 8): 128 accumulators leave room for one weight stage in
    // registers; the next one waits in the wave's LDS stage, two activation stages alternate.
    auto run_full = [&](auto mtc) {
        constexpr int MT = decltype(mtc)::value;
        fl4_t acc[MT][NT];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[a][t] = fl4_t{0.0f, 0.0f, 0.0f, 0.0f};
        uint4 bf[2][NT];
        uint32_t sb[NT];
        const std::integral_constant<int, 1> cs1{};         // scales: fetched per super-step, one ahead
        uint32_t rs_[2], rb_[2], cs_[1], cb_[1];            // next super-step's as loaded; lined up on use
        load_sb(cs1, rs_, rb_, 0);
        load_x(0, xs0);
        issue_w(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0)
        align_sb(cs1, rs_, rb_, cs_, cb_);
        if (nss > 1) load_sb(cs1, rs_, rb_, 1);
        take_w();
        scales_from(cs_[0], cb_[0], 0, sb);
        if (nss > 1) issue_w(1);
        dequant_step(wcur, sb, 0, bf[0]);
        __syncthreads();
        // one super-step: multiplies stage `cur` while stage `nxt` fills
        auto superstep = [&](uint32_t ss, const uint8_t* cur, uint8_t* nxt) {
            if (ss + 1 < nss) load_x(ss + 1, nxt);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (j < 3) dequant_step(wcur, sb, j + 1, bf[(j + 1) & 1]);
                else if (ss + 1 < nss) {
                    // everything in flight has landed: the next activations and weights in LDS,
                    // the next scales in registers
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                    take_w();
                    align_sb(cs1, rs_, rb_, cs_, cb_);
                    if (ss + 2 < nss) load_sb(cs1, rs_, rb_, ss + 2);
                    scales_from(cs_[0], cb_[0], ss + 1, sb);    // ends with lgkmcnt(0): the stage is read before it is refilled
                    if (ss + 2 < nss) issue_w(ss + 2);
                    dequant_step(wcur, sb, 0, bf[0]);
                }
                mfma_step(mtc, acc, cur, j, bf[j & 1]);
            }
            __syncthreads();
        };
        for (uint32_t ss = 0; ss < nss; ss += 2) {
            superstep(ss, xs0, xs1);
            if (ss + 1 < nss) superstep(ss + 1, xs1, xs0);
        }
        epilogue(mtc, acc);
    };

    // ---- short tiles (1 or 2 row tiles).  Little arithmetic per byte of weights: what
    // counts is how much is in flight.  The few accumulators leave registers for a ring of three
    // weight stages (loaded two super-steps ahead), and the three LDS arrays serve as a ring of
    // three activation stages of MT tiles each.  Every wave issues the same MT activation loads
    // per super-step: instruction q = MT wave + e fills quarter q % 4 of tile q / 4.
    auto run_short = [&](auto mtc) {
        constexpr int MT = decltype(mtc)::value;
        fl4_t acc[MT][NT];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[a][t] = fl4_t{0.0f, 0.0f, 0.0f, 0.0f};
        uint32_t xo;                                        // the lane's row of the wave's tile
        {
            const uint32_t row = ((wave * MT) >> 2) * 16 + (lane >> 2);
            const uint32_t m = row < mt.rows ? row : 0;
            const uint32_t src = (DUAL && !p.dense_rows) ? p.pairs[mt.row_start + m].token : mt.row_start + m;
            xo = src * (p.x_stride * 2u) + (uint32_t)((lane & 3) ^ gemm_row_swizzle(lane >> 2)) * 16u;
        }
        auto load_xs = [&](uint32_t ss, uint8_t* stage) {
            const bool tail = odd_tail && ss == nss - 1;
#pragma unroll
            for (int e = 0; e < MT; ++e) {
                const uint32_t q = wave * MT + e;
                uint8_t* dst = stage + (q >> 2) * 4096 + (q & 3) * 1024;
                if (tail && (q & 3) >= 2) *reinterpret_cast<uint4*>(dst + lane * 16) = uint4{0, 0, 0, 0};
                else __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (__attribute__((address_space(3))) void*)dst, 16, xo,
                                                              ss * (GEMM_SK * 2) + (q & 3) * 64, 0, 0);
            }
        };
        struct WReg { uint4 w[NT][WQ]; };
        WReg wr[3];
        auto load_wr = [&](WReg& g, uint32_t ss) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const uint32_t so = wso[t] + ss * (GEMM_SK * BITS / 8);
#pragma unroll
                for (int h = 0; h < WQ; ++h) {
                    const u32x4_t w = __builtin_amdgcn_raw_buffer_load_b128((DUAL && (t & 1)) ? wrsB : wrsA, wv + 16 * h, so, 0);
                    g.w[t][h] = uint4{w.x, w.y, w.z, w.w};
                }
            }
        };
        constexpr int LW = NT * WQ;                         // weight loads of a super-step
        uint4 bf[2][NT];
        uint32_t sb[NT];
        const std::integral_constant<int, 3> cs3{};         // scales: chunks of three super-steps
        uint32_t rs_[4], rb_[4], cs_[3], cb_[3];            // next chunk as loaded, this chunk lined up
        load_sb(cs3, rs_, rb_, 0);
        load_xs(0, xs0);
        load_wr(wr[0], 0);
        if (nss > 1) { load_xs(1, xs1); load_wr(wr[1], 1); }
        align_sb(cs3, rs_, rb_, cs_, cb_);
        if (nss > 3) load_sb(cs3, rs_, rb_, 1);
        scales_from(cs_[0], cb_[0], 0, sb);
        dequant_step(wr[0].w, sb, 0, bf[0]);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        // one super-step (U = its place in its chunk): multiplies stage `cur` from weights `wc`;
        // stage `fill` and weights `wf` take what is needed two super-steps on; `wn` are the
        // weights of the next super-step
        auto superstep = [&](auto uc, uint32_t ss, const uint8_t* cur, uint8_t* fill, const WReg& wc, const WReg& wn, WReg& wf) {
            constexpr int U = decltype(uc)::value;
            if (ss + 2 < nss) { load_xs(ss + 2, fill); load_wr(wf, ss + 2); }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (j < 3) dequant_step(wc.w, sb, j + 1, bf[(j + 1) & 1]);
                else if (ss + 1 < nss) {
                    if (U == 2) {
                        align_sb(cs3, rs_, rb_, cs_, cb_);
                        if (ss + 4 < nss) load_sb(cs3, rs_, rb_, (ss + 4) / 3);
                    }
                    scales_from(cs_[(U + 1) % 3], cb_[(U + 1) % 3], ss + 1, sb);
                    dequant_step(wn.w, sb, 0, bf[0]);
                }
                mfma_step(mtc, acc, cur, j, bf[j & 1]);
            }
            // The next activation stage was requested a super-step ago; at least the MT + LW
            // requests from the start of this super-step are younger.  Near the end, or where a
            // stage took zeros instead of loads, fewer were issued and more is waited for.
            if (ss + 2 < nss && !(odd_tail && ss + 2 == nss - 1)) __builtin_amdgcn_s_waitcnt(gemm_vmcnt(MT + LW));
            else __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        };
        for (uint32_t ss = 0; ss < nss; ss += 3) {
            superstep(std::integral_constant<int, 0>{}, ss, xs0, ws, wr[0], wr[1], wr[2]);
            if (ss + 1 < nss) superstep(std::integral_constant<int, 1>{}, ss + 1, xs1, xs0, wr[1], wr[2], wr[0]);
            if (ss + 2 < nss) superstep(std::integral_constant<int, 2>{}, ss + 2, ws, xs1, wr[2], wr[0], wr[1]);
        }
        epilogue(mtc, acc);
    };
    // ---- short tiles whose scales and biases fit the second activation array: rows of scales
    // that are a multiple of 16 bytes (K a multiple of 512) and at most 16 KB per array for the
    // block's columns.  Fetched lane by lane the scales arrive 16 bytes from each of 64 rows per
    // instruction; here each wave fetches the whole rows of its 16 NT columns once, contiguously,
    // into a table in LDS, and a super-step reads its dword (two groups) per tile from there.
    // The activations then alternate between the first activation array and the weight stage
    // array (fetched one super-step ahead); the weights keep their ring of three register stages.
    auto run_short_tab = [&](auto mtc) {
        constexpr int MT = decltype(mtc)::value;
        fl4_t acc[MT][NT];
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[a][t] = fl4_t{0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t g2 = groups * 2u;                    // bytes per row of scales
        uint8_t* tab_s = xs1;
        uint8_t* tab_b = xs1 + GEMM_XBUF / 2;
        {
            const uint32_t ppr = g2 / 16u, total = NT * 16u * ppr;      // 16-byte pieces per row, per wave
            for (uint32_t i = 0; i * 64u < total; ++i) {
                const uint32_t q = i * 64u + lane;
                const uint32_t row = q / ppr, piece = q % ppr;          // row = 16 t + column of the tile
                const uint32_t t = row >> 4, c16 = row & 15u;
                uint32_t c = DUAL ? n0 + wave * (8 * NT) + (t >> 1) * 16 + c16 : n0 + wave * (16 * NT) + t * 16 + c16;
                c = min(c, p.N - 1) * g2 + piece * 16u;
                const uint32_t so = (DUAL ? (uint32_t)((t & 1) ? p.sB : p.sA) : 0u) + c;
                const uint32_t bo = (DUAL ? (uint32_t)((t & 1) ? p.bB : p.bA) : 0u) + c;
                const uint32_t at = wave * (NT * 16u) * g2 + i * 1024u;
                if (q < total) {
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(s_rs, (__attribute__((address_space(3))) void*)(tab_s + at), 16, so, 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rs, (__attribute__((address_space(3))) void*)(tab_b + at), 16, bo, 0, 0, 0);
                }
            }
        }
        const uint32_t tb = (wave * (NT * 16u) + li) * g2;  // the lane's column of tile 0 in the tables
        auto fetch_sb = [&](uint32_t ss, uint32_t* ds, uint32_t* db) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                ds[t] = *reinterpret_cast<const uint32_t*>(tab_s + tb + t * 16u * g2 + ss * 4u);
                db[t] = *reinterpret_cast<const uint32_t*>(tab_b + tb + t * 16u * g2 + ss * 4u);
            }
        };
        auto pack_sb = [&](const uint32_t* ds, const uint32_t* db, uint32_t* sb) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
                sb[t] = (lq >> 1) ? __builtin_amdgcn_perm(ds[t], db[t], 0x07060302u)
                                  : __builtin_amdgcn_perm(ds[t], db[t], 0x05040100u);
        };
        uint32_t xo;                                        // the lane's row of the wave's tile
        {
            const uint32_t row = ((wave * MT) >> 2) * 16 + (lane >> 2);
            const uint32_t m = row < mt.rows ? row : 0;
            const uint32_t src = (DUAL && !p.dense_rows) ? p.pairs[mt.row_start + m].token : mt.row_start + m;
            xo = src * (p.x_stride * 2u) + (uint32_t)((lane & 3) ^ gemm_row_swizzle(lane >> 2)) * 16u;
        }
        auto load_xs = [&](uint32_t ss, uint8_t* stage) {
#pragma unroll
            for (int e = 0; e < MT; ++e) {
                const uint32_t q = wave * MT + e;
                uint8_t* dst = stage + (q >> 2) * 4096 + (q & 3) * 1024;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (__attribute__((address_space(3))) void*)dst, 16, xo,
                                                         ss * (GEMM_SK * 2) + (q & 3) * 64, 0, 0);
            }
        };
        struct WReg { uint4 w[NT][WQ]; };
        WReg wr[3];
        auto load_wr = [&](WReg& g, uint32_t ss) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const uint32_t so = wso[t] + ss * (GEMM_SK * BITS / 8);
#pragma unroll
                for (int h = 0; h < WQ; ++h) {
                    const u32x4_t w = __builtin_amdgcn_raw_buffer_load_b128((DUAL && (t & 1)) ? wrsB : wrsA, wv + 16 * h, so, 0);
                    g.w[t][h] = uint4{w.x, w.y, w.z, w.w};
                }
            }
        };
        constexpr int LW = NT * WQ;                         // weight loads of a super-step
        uint4 bf[2][NT];
        uint32_t sb[NT];
        load_xs(0, xs0);
        load_wr(wr[0], 0);
        if (nss > 1) load_wr(wr[1], 1);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        {
            uint32_t ds[NT], db[NT];
            fetch_sb(0, ds, db);
            pack_sb(ds, db, sb);
        }
        dequant_step(wr[0].w, sb, 0, bf[0]);
        // one super-step: multiplies stage `cur` from weights `wc`; stage `nxt` takes the next
        // super-step's activations, `wf` the weights needed two super-steps on; `wn` are the
        // weights of the next super-step
        auto superstep = [&](uint32_t ss, const uint8_t* cur, uint8_t* nxt, const WReg& wc, const WReg& wn, WReg& wf) {
            if (ss + 1 < nss) load_xs(ss + 1, nxt);
            if (ss + 2 < nss) load_wr(wf, ss + 2);
            uint32_t ds[NT], db[NT];
            if (ss + 1 < nss) fetch_sb(ss + 1, ds, db);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (j < 3) dequant_step(wc.w, sb, j + 1, bf[(j + 1) & 1]);
                else if (ss + 1 < nss) {
                    pack_sb(ds, db, sb);
                    dequant_step(wn.w, sb, 0, bf[0]);
                }
                mfma_step(mtc, acc, cur, j, bf[j & 1]);
            }
            // the next activation stage was requested at the top; only the LW weight requests
            // that followed it may still be under way
            if (ss + 2 < nss) __builtin_amdgcn_s_waitcnt(gemm_vmcnt(LW));
            else __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        };
        for (uint32_t ss = 0; ss < nss; ss += 6) {
            superstep(ss, xs0, ws, wr[0], wr[1], wr[2]);
            if (ss + 1 < nss) superstep(ss + 1, ws, xs0, wr[1], wr[2], wr[0]);
            if (ss + 2 < nss) superstep(ss + 2, xs0, ws, wr[2], wr[0], wr[1]);
            if (ss + 3 < nss) superstep(ss + 3, ws, xs0, wr[0], wr[1], wr[2]);
            if (ss + 4 < nss) superstep(ss + 4, xs0, ws, wr[1], wr[2], wr[0]);
            if (ss + 5 < nss) superstep(ss + 5, ws, xs0, wr[2], wr[0], wr[1]);
        }
        epilogue(mtc, acc);
    };
    // K a multiple of 512 has no half super-step at the end either
    const bool tab_ok = (groups % 8u) == 0 && 64u * NT * groups * 2u <= GEMM_XBUF / 2;
    // (three and four row tiles through the table body: 256 experts x 48 rows 120 -> 100 us, x 64 rows 122 -> 100 us)
    if (live_mt > 4) run_full(std::integral_constant<int, 8>{});
    else if (live_mt > 2) { if (tab_ok) run_short_tab(std::integral_constant<int, 4>{}); else run_full(std::integral_constant<int, 4>{}); }
    else if (live_mt > 1) { if (tab_ok) run_short_tab(std::integral_constant<int, 2>{}); else run_short(std::integral_constant<int, 2>{}); }
    else { if (tab_ok) run_short_tab(std::integral_constant<int, 1>{}); else run_short(std::integral_constant<int, 1>{}); }
}

// y[t, :] = rows[t, :] scaled by 1 / (1 + exp(-gate_logit[t])) where a gate is given (the shared
// expert's scalar gate, utility.metal:61-70), else copied: rows are 16-bit activations [tokens, d].
template <int ACT>
__global__ __launch_bounds__(256) void gate_rows_kernel(const uint16_t* rows, const float* gate_logit, uint16_t* y,
                                                       uint32_t tokens, uint32_t d, uint32_t y_stride) {
    const uint32_t t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    float v = act_to_f32<ACT>(rows[(size_t)t * d + c]);
    if (gate_logit) v = __fdiv_rn(v, __fadd_rn(1.0f, expf(-gate_logit[t])));
    y[(size_t)t * y_stride + c] = f32_to_act<ACT>(v);
}

// The same, eight values (16 bytes) per thread: d a multiple of 8, rows and y rows 16-byte aligned.
template <int ACT>
__global__ __launch_bounds__(256) void gate_rows8_kernel(const uint16_t* rows, const float* gate_logit, uint16_t* y,
                                                        uint32_t tokens, uint32_t d, uint32_t y_stride) {
    const uint32_t t = blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 8u;
    if (c >= d) return;
    const uint4 v = *reinterpret_cast<const uint4*>(rows + (size_t)t * d + c);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float den = 1.0f;
    if (gate_logit) den = __fadd_rn(1.0f, expf(-gate_logit[t]));
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float lo, hi;
        act2_to_f32<ACT>(w[j], lo, hi);
        if (gate_logit) { lo = __fdiv_rn(lo, den); hi = __fdiv_rn(hi, den); }
        r[j] = (uint32_t)f32_to_act<ACT>(lo) | ((uint32_t)f32_to_act<ACT>(hi) << 16);
    }
    *reinterpret_cast<uint4*>(y + (size_t)t * y_stride + c) = uint4{r[0], r[1], r[2], r[3]};
}

// ---- combine (prefill.metal:437-458) -------------------------------------------------------
// h2[t, d] = sum over ranks in rank order of fma(w[t, r], partial[t, r, d], acc).  VEC = 8:
// sixteen bytes of a row per thread (rows 16-byte aligned); VEC = 2: any even d.
template <int ACT, int VEC>
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const void* partials, const uint16_t* w, void* h2,
                                                            uint32_t tokens, uint32_t top_k, uint32_t d,
                                                            uint32_t h2_stride) {
    const uint32_t t = blockIdx.y;
    const uint32_t c = (blockIdx.x * 256 + threadIdx.x) * VEC;
    if (c >= d) return;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.0f;
    const uint16_t* src = (const uint16_t*)partials + (size_t)t * top_k * d + c;
    for (uint32_t r = 0; r < top_k; ++r) {
        const float wr = f16_to_f32(w[(size_t)t * top_k + r]);
        uint32_t v[VEC / 2];
        if (VEC == 8) {
            const uint4 q = *reinterpret_cast<const uint4*>(src + (size_t)r * d);
            v[0] = q.x; v[VEC == 8 ? 1 : 0] = q.y; v[VEC == 8 ? 2 : 0] = q.z; v[VEC == 8 ? 3 : 0] = q.w;
        } else {
            v[0] = *reinterpret_cast<const uint32_t*>(src + (size_t)r * d);
        }
#pragma unroll
        for (int j = 0; j < VEC / 2; ++j) {
            float lo, hi;
            act2_to_f32<ACT>(v[j], lo, hi);
            acc[2 * j] = fmaf(wr, lo, acc[2 * j]);
            acc[2 * j + 1] = fmaf(wr, hi, acc[2 * j + 1]);
        }
    }
    uint16_t* o = (uint16_t*)h2 + (size_t)t * h2_stride + c;
    if (VEC == 8) {
        uint4 q;
        q.x = f32_to_act<ACT>(acc[0]) | (uint32_t)f32_to_act<ACT>(acc[1]) << 16;
        q.y = f32_to_act<ACT>(acc[VEC == 8 ? 2 : 0]) | (uint32_t)f32_to_act<ACT>(acc[VEC == 8 ? 3 : 0]) << 16;
        q.z = f32_to_act<ACT>(acc[VEC == 8 ? 4 : 0]) | (uint32_t)f32_to_act<ACT>(acc[VEC == 8 ? 5 : 0]) << 16;
        q.w = f32_to_act<ACT>(acc[VEC == 8 ? 6 : 0]) | (uint32_t)f32_to_act<ACT>(acc[VEC == 8 ? 7 : 0]) << 16;
        *reinterpret_cast<uint4*>(o) = q;
    } else {
        o[0] = f32_to_act<ACT>(acc[0]);
        o[1] = f32_to_act<ACT>(acc[1]);
    }
}

}  // namespace nvmai
