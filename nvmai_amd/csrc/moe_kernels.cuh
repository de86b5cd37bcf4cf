// Decode-side kernels of the quantized MoE path: affine-row GEMV engines
// (gate/up SwiGLU and down), router logits, device top-k + expert work list,
// weighted combine, and the affine group-64 quantizer.  gfx950, wave64.
#pragma once

#include "common.cuh"

namespace nvmai {

// Where an expert blob lives: a resident pool (base + index * stride) or one of
// nine pointers passed by value (the reference's RoutedBlobs table,
// moe.metal:153-155, plus one slot for the shared expert).
struct BlobSource {
    const uint8_t* pool_base;
    uint64_t pool_stride;
    const uint8_t* slot[9];
};
#define NVMAI_SLOT_FLAG 0x80000000u

__device__ __forceinline__ const uint8_t* blob_ptr(const BlobSource& src, uint32_t expert) {
    return (expert & NVMAI_SLOT_FLAG) ? src.slot[expert & 0xFu]
                                      : src.pool_base + (uint64_t)expert * src.pool_stride;
}

// One unit of expert work: up to TOK (token, slot) pairs routed to one expert.
struct WorkEntry {
    uint32_t expert;      // pool index, or NVMAI_SLOT_FLAG | slot
    uint32_t pair_start;  // into pair_token / pair_id
    uint32_t pair_count;  // 1..MAX_TOK
    uint32_t reserved;
};
constexpr int MAX_TOK = 4;

struct RowsParams {
    BlobSource src;
    const WorkEntry* entries;
    const uint32_t* n_entries;   // device counter
    const uint32_t* pair_in;     // input row per pair (token, or act row)
    const uint32_t* pair_out;    // output row per pair
    int64_t wA, sA, bA;          // byte offsets of matrix A inside the blob
    int64_t wB, sB, bB;          // matrix B (DUAL only: up projection)
    const void* x;               // inputs: 16-bit activations or fp32
    uint32_t x_stride;           // elements between input rows
    float* out;                  // fp32 [out rows, rows]
    uint32_t out_stride;
    uint32_t rows, n;            // matrix shape [rows, n]
    uint32_t blocks_per_entry;
};

// ---- input staging ----------------------------------------------------------
// Load EPC consecutive inputs starting at element e0 of one input row as floats.
template <int ACT, bool XF32, int EPC>
__device__ __forceinline__ void load_x(const void* x, size_t row_off, uint32_t e0, float* dst) {
    if (XF32) {
        const float4* p = reinterpret_cast<const float4*>((const float*)x + row_off + e0);
#pragma unroll
        for (int i = 0; i < EPC / 4; ++i) {
            float4 v = p[i];
            dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>((const uint16_t*)x + row_off + e0);
#pragma unroll
        for (int i = 0; i < EPC / 8; ++i) {
            uint4 v = p[i];
            act2_to_f32<ACT>(v.x, dst[8 * i], dst[8 * i + 1]);
            act2_to_f32<ACT>(v.y, dst[8 * i + 2], dst[8 * i + 3]);
            act2_to_f32<ACT>(v.z, dst[8 * i + 4], dst[8 * i + 5]);
            act2_to_f32<ACT>(v.w, dst[8 * i + 6], dst[8 * i + 7]);
        }
    }
}

// ---- fast engine ------------------------------------------------------------
// A row of n codes is n*BITS/128 chunks of 16 bytes.  SEG lanes share a row
// (SEG*NCH chunks), so one wave covers 64/SEG rows per load instruction and
// every load instruction moves 1 KiB of contiguous weights.  Lane inputs are
// the same columns for every row, so they sit in registers for the whole block.
// Per chunk the arithmetic is the reference's factoring (nvmai_kernels.h:19-21):
// acc += scale * sum(q*x) + bias * sum(x), with sum(x) hoisted out of the row
// loop as int4_affine_gemv.c:41-53 does.
template <int ACT, int BITS, int SEG, int NCH, int TOK, bool DUAL, bool XF32, int RPI, int ITERS>
__device__ __forceinline__ void expert_rows_body(const RowsParams& p, const WorkEntry& we, uint32_t rb) {
    constexpr int EPC = Chunk<BITS>::elems;
    constexpr int RPL = 64 / SEG;                 // rows per load instruction
    constexpr int ROWS_WAVE = RPL * RPI * ITERS;
    const uint8_t* blob = blob_ptr(p.src, we.expert);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int seg_id = lane / SEG, sl = lane % SEG;
    const uint32_t groups = p.n / NVMAI_GROUP;
    const uint32_t row_bytes = p.n * BITS / 8;

    float xr[TOK][NCH][EPC];
    float xs[TOK][NCH];
    uint32_t out_row[TOK];
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
        const bool live = (uint32_t)t < we.pair_count;
        const uint32_t pi = we.pair_start + (live ? t : 0);
        const size_t in_off = (size_t)p.pair_in[pi] * p.x_stride;
        out_row[t] = p.pair_out[pi];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            load_x<ACT, XF32, EPC>(p.x, in_off, (uint32_t)(sl + c * SEG) * EPC, xr[t][c]);
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < EPC; ++j) {
                if (!live) xr[t][c][j] = 0.0f;
                s += xr[t][c][j];
            }
            xs[t][c] = s;
        }
    }

    const uint8_t* WA = blob + p.wA;
    const uint16_t* SA = reinterpret_cast<const uint16_t*>(blob + p.sA);
    const uint16_t* BA = reinterpret_cast<const uint16_t*>(blob + p.bA);
    const uint8_t* WB = DUAL ? blob + p.wB : nullptr;
    const uint16_t* SB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.sB) : nullptr;
    const uint16_t* BB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.bB) : nullptr;

    const uint32_t row_base = (rb * 4 + wave) * ROWS_WAVE;
#pragma unroll 1
    for (int it = 0; it < ITERS; ++it) {
        uint4 qa[RPI][NCH], qb[RPI][NCH];
        uint16_t sa[RPI][NCH], ba[RPI][NCH], sb[RPI][NCH], bb[RPI][NCH];
        uint32_t rows_i[RPI];
        // issue every load of this iteration before the first use
#pragma unroll
        for (int i = 0; i < RPI; ++i) {
            const uint32_t row = row_base + (it * RPI + i) * RPL + seg_id;
            rows_i[i] = row;
            const uint32_t r = row < p.rows ? row : p.rows - 1;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const uint32_t chunk = sl + c * SEG;
                const uint32_t g = chunk * EPC / NVMAI_GROUP;
                qa[i][c] = *reinterpret_cast<const uint4*>(WA + (size_t)r * row_bytes + chunk * 16);
                sa[i][c] = SA[(size_t)r * groups + g];
                ba[i][c] = BA[(size_t)r * groups + g];
                if (DUAL) {
                    qb[i][c] = *reinterpret_cast<const uint4*>(WB + (size_t)r * row_bytes + chunk * 16);
                    sb[i][c] = SB[(size_t)r * groups + g];
                    bb[i][c] = BB[(size_t)r * groups + g];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < RPI; ++i) {
            float accA[TOK], accB[TOK];
#pragma unroll
            for (int t = 0; t < TOK; ++t) { accA[t] = 0.0f; accB[t] = 0.0f; }
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                float q[EPC];
                unpack_chunk<BITS>(qa[i][c], q);
                const float s = bf16_to_f32(sa[i][c]), b = bf16_to_f32(ba[i][c]);
#pragma unroll
                for (int t = 0; t < TOK; ++t) {
                    float dot = 0.0f;
#pragma unroll
                    for (int j = 0; j < EPC; ++j) dot = fmaf(q[j], xr[t][c][j], dot);
                    accA[t] = fmaf(s, dot, accA[t]);
                    accA[t] = fmaf(b, xs[t][c], accA[t]);
                }
                if (DUAL) {
                    unpack_chunk<BITS>(qb[i][c], q);
                    const float s2 = bf16_to_f32(sb[i][c]), b2 = bf16_to_f32(bb[i][c]);
#pragma unroll
                    for (int t = 0; t < TOK; ++t) {
                        float dot = 0.0f;
#pragma unroll
                        for (int j = 0; j < EPC; ++j) dot = fmaf(q[j], xr[t][c][j], dot);
                        accB[t] = fmaf(s2, dot, accB[t]);
                        accB[t] = fmaf(b2, xs[t][c], accB[t]);
                    }
                }
            }
            const bool writer = seg_result_lane<SEG>(lane) && rows_i[i] < p.rows;
#pragma unroll
            for (int t = 0; t < TOK; ++t) {
                float a = seg_reduce_sum<SEG>(accA[t]);
                float v = a;
                if (DUAL) {
                    float u = seg_reduce_sum<SEG>(accB[t]);
                    v = silu(a) * u;      // moe.metal:134-139 (silu branch), CPUExpertFFN.swift:122-124
                }
                if (writer && (uint32_t)t < we.pair_count)
                    p.out[(size_t)out_row[t] * p.out_stride + rows_i[i]] = v;
            }
        }
    }
}

// MAXTOK = 1: single-input launches.  MAXTOK = 4: the body is chosen by the
// entry's pair count (uniform per block), so an expert routed to by one token
// does not pay for four.
template <int ACT, int BITS, int SEG, int NCH, int MAXTOK, bool DUAL, bool XF32, int RPI, int ITERS>
__global__ __launch_bounds__(256) void expert_rows_fast(RowsParams p) {
    const uint32_t entry = blockIdx.x / p.blocks_per_entry;
    if (entry >= *p.n_entries) return;
    const uint32_t rb = blockIdx.x % p.blocks_per_entry;
    const WorkEntry we = p.entries[entry];
    if (MAXTOK == 1 || we.pair_count == 1)
        expert_rows_body<ACT, BITS, SEG, NCH, 1, DUAL, XF32, RPI, ITERS>(p, we, rb);
    else if (we.pair_count == 2)
        expert_rows_body<ACT, BITS, SEG, NCH, 2, DUAL, XF32, RPI, ITERS>(p, we, rb);
    else
        expert_rows_body<ACT, BITS, SEG, NCH, 4, DUAL, XF32, RPI, ITERS>(p, we, rb);
}

// ---- generic engine -----------------------------------------------------------
// Any n that is a multiple of 64: one wave per row, lanes stride over chunks and
// re-read the inputs from memory.  Used for shapes without a fast instantiation.
template <int ACT, int BITS, bool DUAL, bool XF32>
__global__ __launch_bounds__(256) void expert_rows_generic(RowsParams p) {
    constexpr int EPC = Chunk<BITS>::elems;
    constexpr int ROWS_WAVE = 4;
    const uint32_t entry = blockIdx.x / p.blocks_per_entry;
    if (entry >= *p.n_entries) return;
    const uint32_t rb = blockIdx.x % p.blocks_per_entry;
    const WorkEntry we = p.entries[entry];
    const uint8_t* blob = blob_ptr(p.src, we.expert);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t groups = p.n / NVMAI_GROUP;
    const uint32_t row_bytes = p.n * BITS / 8;
    const uint32_t chunks = row_bytes / 16;
    const uint8_t* WA = blob + p.wA;
    const uint16_t* SA = reinterpret_cast<const uint16_t*>(blob + p.sA);
    const uint16_t* BA = reinterpret_cast<const uint16_t*>(blob + p.bA);
    const uint8_t* WB = DUAL ? blob + p.wB : nullptr;
    const uint16_t* SB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.sB) : nullptr;
    const uint16_t* BB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.bB) : nullptr;

    for (int i = 0; i < ROWS_WAVE; ++i) {
        const uint32_t row = (rb * 4 + wave) * ROWS_WAVE + i;
        if (row >= p.rows) return;     // uniform per wave
        float accA[MAX_TOK], accB[MAX_TOK];
#pragma unroll
        for (int t = 0; t < MAX_TOK; ++t) { accA[t] = 0.0f; accB[t] = 0.0f; }
        for (uint32_t chunk = lane; chunk < chunks; chunk += 64) {
            const uint32_t g = chunk * EPC / NVMAI_GROUP;
            float qa[EPC], qb[EPC];
            unpack_chunk<BITS>(*reinterpret_cast<const uint4*>(WA + (size_t)row * row_bytes + chunk * 16), qa);
            const float sa = bf16_to_f32(SA[(size_t)row * groups + g]);
            const float ba = bf16_to_f32(BA[(size_t)row * groups + g]);
            float sb = 0.0f, bb = 0.0f;
            if (DUAL) {
                unpack_chunk<BITS>(*reinterpret_cast<const uint4*>(WB + (size_t)row * row_bytes + chunk * 16), qb);
                sb = bf16_to_f32(SB[(size_t)row * groups + g]);
                bb = bf16_to_f32(BB[(size_t)row * groups + g]);
            }
#pragma unroll
            for (int t = 0; t < MAX_TOK; ++t) {
                if ((uint32_t)t >= we.pair_count) break;
                float xv[EPC];
                load_x<ACT, XF32, EPC>(p.x, (size_t)p.pair_in[we.pair_start + t] * p.x_stride, chunk * EPC, xv);
                float dot = 0.0f, xsum = 0.0f, dot2 = 0.0f;
#pragma unroll
                for (int j = 0; j < EPC; ++j) {
                    dot = fmaf(qa[j], xv[j], dot);
                    if (DUAL) dot2 = fmaf(qb[j], xv[j], dot2);
                    xsum += xv[j];
                }
                accA[t] = fmaf(sa, dot, accA[t]);
                accA[t] = fmaf(ba, xsum, accA[t]);
                if (DUAL) {
                    accB[t] = fmaf(sb, dot2, accB[t]);
                    accB[t] = fmaf(bb, xsum, accB[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MAX_TOK; ++t) {
            if ((uint32_t)t >= we.pair_count) break;
            float a = seg_reduce_sum<64>(accA[t]);
            float v = a;
            if (DUAL) v = silu(a) * seg_reduce_sum<64>(accB[t]);
            if (lane == 63)
                p.out[(size_t)p.pair_out[we.pair_start + t] * p.out_stride + row] = v;
        }
    }
}

// ---- router logits --------------------------------------------------------------
// Rows in "router format": kind 8 / 4 = affine codes + bf16 scale/bias per group of
// 64, kind 16 = dense bf16.  One half-wave (32 lanes) owns one row.  Lane l owns
// the 16-byte chunks l, l+32, ...; inside a chunk dot = fma(q, x, dot) and
// xs = xs + x run in element order, then acc = fma(s, dot, acc), acc = fma(b, xs,
// acc); the 32 accumulators are summed by an xor butterfly 16, 8, 4, 2, 1.  This
// order is part of the contract: routing indices are compared bit-exactly against
// a CPU run of the same order.
struct RowsDesc {
    const void* w;
    const uint16_t* s;
    const uint16_t* b;
    int kind;     // 4, 8, 16; 0 = absent
};

struct RouterParams {
    RowsDesc router;
    RowsDesc gate;                 // optional single row appended after the experts
    const void* x;                 // [tokens, x_stride] activations
    const uint16_t* eff_scale;     // optional bf16 [d]
    uint32_t x_stride, tokens, num_experts, d;
    float* logits;                 // [tokens, num_experts]
    float* gate_logit;             // [tokens]
};

template <int ACT>
__device__ __forceinline__ float router_x(const RouterParams& p, size_t row_off, uint32_t e) {
    float v = act_to_f32<ACT>(((const uint16_t*)p.x)[row_off + e]);
    if (p.eff_scale) v = __fmul_rn(v, bf16_to_f32(p.eff_scale[e]));
    return v;
}

template <int ACT>
__device__ float router_row_dot(const RouterParams& p, const RowsDesc& r, uint32_t row,
                                size_t x_off, int hl) {
    float acc = 0.0f;
    if (r.kind == 16) {
        const uint32_t chunks = p.d / 8;
        const uint16_t* wr = (const uint16_t*)r.w + (size_t)row * p.d;
        for (uint32_t c = hl; c < chunks; c += 32) {
            uint4 raw = *reinterpret_cast<const uint4*>(wr + c * 8);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = fmaf(__uint_as_float(words[j] << 16), router_x<ACT>(p, x_off, c * 8 + 2 * j), acc);
                acc = fmaf(__uint_as_float(words[j] & 0xFFFF0000u), router_x<ACT>(p, x_off, c * 8 + 2 * j + 1), acc);
            }
        }
    } else {
        const int epc = r.kind == 8 ? 16 : 32;
        const uint32_t chunks = p.d / epc;
        const uint32_t groups = p.d / NVMAI_GROUP;
        const uint8_t* wr = (const uint8_t*)r.w + (size_t)row * (p.d * r.kind / 8);
        for (uint32_t c = hl; c < chunks; c += 32) {
            const uint4 raw = *reinterpret_cast<const uint4*>(wr + c * 16);
            const uint32_t g = c * epc / NVMAI_GROUP;
            const float s = bf16_to_f32(r.s[(size_t)row * groups + g]);
            const float b = bf16_to_f32(r.b[(size_t)row * groups + g]);
            float q[32];
            if (r.kind == 8) unpack_chunk<8>(raw, q); else unpack_chunk<4>(raw, q);
            float dot = 0.0f, xs = 0.0f;
            for (int j = 0; j < epc; ++j) {
                const float xv = router_x<ACT>(p, x_off, c * epc + j);
                dot = fmaf(q[j], xv, dot);
                xs = __fadd_rn(xs, xv);
            }
            acc = fmaf(s, dot, acc);
            acc = fmaf(b, xs, acc);
        }
    }
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) acc = __fadd_rn(acc, shfl_xor_f(acc, off));
    return acc;
}

constexpr int ROUTER_TOK = 4;   // tokens per block in y

template <int ACT>
__global__ __launch_bounds__(256) void router_logits_kernel(RouterParams p) {
    const int hw = threadIdx.x >> 5, hl = threadIdx.x & 31;
    const uint32_t row = blockIdx.x * 8 + hw;
    const uint32_t total_rows = p.num_experts + (p.gate.kind ? 1u : 0u);
    if (row >= total_rows) return;                   // uniform per half-wave
    const bool is_gate = row >= p.num_experts;
    for (uint32_t t = blockIdx.y * ROUTER_TOK; t < min(p.tokens, (blockIdx.y + 1) * ROUTER_TOK); ++t) {
        const size_t x_off = (size_t)t * p.x_stride;
        float v = is_gate ? router_row_dot<ACT>(p, p.gate, 0, x_off, hl)
                          : router_row_dot<ACT>(p, p.router, row, x_off, hl);
        if (hl == 0) {
            if (is_gate) p.gate_logit[t] = v;
            else p.logits[(size_t)t * p.num_experts + row] = v;
        }
    }
}

// ---- top-k select + softmax over the selected ------------------------------------
// One wave per token.  Selection equals a stable sort by (score desc, index asc)
// (moe.metal:233-285).  Weights: ex_i = exp(s_i - s_0), sum in slot order,
// w_i = ex_i / sum * per_expert_scale, stored as fp16 (moe.metal:268-284).
constexpr int TOPK_MAX_PER_LANE = 8;   // num_experts <= 512

struct SelectParams {
    const float* logits;              // [tokens, num_experts]
    const uint16_t* per_expert_scale; // optional bf16
    uint32_t tokens, num_experts, top_k;
    uint32_t* out_idx;                // [tokens, top_k]
    uint16_t* out_w;                  // fp16 [tokens, top_k]
};

__device__ __forceinline__ bool better(float v, uint32_t i, float v2, uint32_t i2) {
    return v > v2 || (v == v2 && i < i2);
}

__device__ void select_topk_wave(const SelectParams& p, uint32_t t, int lane) {
    float val[TOPK_MAX_PER_LANE];
    bool taken[TOPK_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < TOPK_MAX_PER_LANE; ++j) {
        const uint32_t e = lane + 64 * j;
        val[j] = e < p.num_experts ? p.logits[(size_t)t * p.num_experts + e] : 0.0f;
        taken[j] = e >= p.num_experts;
    }
    float my_score = 0.0f;
    uint32_t my_idx = 0;
    for (uint32_t round = 0; round < p.top_k; ++round) {
        float bv = -INFINITY;
        uint32_t bi = 0xFFFFFFFFu;
#pragma unroll
        for (int j = 0; j < TOPK_MAX_PER_LANE; ++j) {
            const uint32_t e = lane + 64 * j;
            if (!taken[j] && (bi == 0xFFFFFFFFu || better(val[j], e, bv, bi))) { bv = val[j]; bi = e; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = shfl_xor_f(bv, off);
            const uint32_t oi = shfl_xor_u(bi, off);
            if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || better(ov, oi, bv, bi))) { bv = ov; bi = oi; }
        }
        if (bi == 0xFFFFFFFFu) { bi = 0; bv = -INFINITY; }   // fewer candidates than k
#pragma unroll
        for (int j = 0; j < TOPK_MAX_PER_LANE; ++j)
            if ((uint32_t)(lane + 64 * j) == bi) taken[j] = true;
        if ((uint32_t)lane == round) { my_score = bv; my_idx = bi; }
    }
    const float max_s = readlane_f(my_score, 0);
    const float ex = expf(my_score - max_s);
    float sum = 0.0f;
    for (uint32_t i = 0; i < p.top_k; ++i) sum = __fadd_rn(sum, __shfl(ex, (int)i, 64));
    if ((uint32_t)lane < p.top_k) {
        const float gain = p.per_expert_scale ? bf16_to_f32(p.per_expert_scale[my_idx]) : 1.0f;
        const float w = __fmul_rn(__fdiv_rn(ex, sum), gain);
        p.out_idx[(size_t)t * p.top_k + lane] = my_idx;
        p.out_w[(size_t)t * p.top_k + lane] = f32_to_f16(w);
    }
}

__global__ __launch_bounds__(256) void select_topk_kernel(SelectParams p) {
    const uint32_t t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t < p.tokens) select_topk_wave(p, t, threadIdx.x & 63);
}

// ---- decode work list --------------------------------------------------------------
// Groups the (token, slot) pairs of a small decode batch by expert so that each
// distinct expert is streamed once, and appends the shared expert over all
// tokens.  One block; thread e owns expert e.  Pair order inside an expert is
// (token, slot) ascending, which makes the result deterministic.
struct GroupParams {
    const uint32_t* idx;       // [tokens, top_k]
    uint32_t tokens, top_k, num_experts;
    uint32_t tok_per_entry;    // 1..MAX_TOK
    int has_shared;
    WorkEntry* entries;
    uint32_t* n_entries;       // [0] = entries, [1] = distinct experts
    uint32_t* pair_token;      // input row per pair for phase 1
    uint32_t* pair_id;         // act / partial row per pair
};

__global__ __launch_bounds__(1024) void group_decode_kernel(GroupParams p) {
    extern __shared__ uint32_t lds[];
    uint32_t* s_idx = lds;                                // tokens*top_k
    uint32_t* s_scan = lds + p.tokens * p.top_k;          // 2 * blockDim
    const uint32_t tid = threadIdx.x, n_pairs = p.tokens * p.top_k;
    for (uint32_t i = tid; i < n_pairs; i += blockDim.x) s_idx[i] = p.idx[i];
    __syncthreads();
    uint32_t cnt = 0;
    if (tid < p.num_experts)
        for (uint32_t i = 0; i < n_pairs; ++i) cnt += (s_idx[i] == tid);
    const uint32_t ent = (cnt + p.tok_per_entry - 1) / p.tok_per_entry;
    // inclusive scans of pair counts and entry counts (Hillis-Steele in LDS)
    uint32_t* sc_pairs = s_scan;
    uint32_t* sc_ent = s_scan + blockDim.x;
    sc_pairs[tid] = cnt;
    sc_ent[tid] = ent;
    __syncthreads();
    for (uint32_t off = 1; off < blockDim.x; off <<= 1) {
        uint32_t a = 0, b = 0;
        if (tid >= off) { a = sc_pairs[tid - off]; b = sc_ent[tid - off]; }
        __syncthreads();
        sc_pairs[tid] += a;
        sc_ent[tid] += b;
        __syncthreads();
    }
    const uint32_t pair_start = sc_pairs[tid] - cnt, ent_start = sc_ent[tid] - ent;
    const uint32_t total_ent = sc_ent[blockDim.x - 1];
    if (cnt) {
        uint32_t k = 0;
        for (uint32_t i = 0; i < n_pairs; ++i) {
            if (s_idx[i] != tid) continue;
            if (k % p.tok_per_entry == 0) {
                WorkEntry we;
                we.expert = tid;
                we.pair_start = pair_start + k;
                we.pair_count = min(p.tok_per_entry, cnt - k);
                we.reserved = 0;
                p.entries[ent_start + k / p.tok_per_entry] = we;
            }
            p.pair_token[pair_start + k] = i / p.top_k;
            p.pair_id[pair_start + k] = i;
            ++k;
        }
    }
    // distinct experts = number of threads with cnt > 0
    __syncthreads();
    sc_pairs[tid] = cnt ? 1u : 0u;
    __syncthreads();
    for (uint32_t off = blockDim.x / 2; off > 0; off >>= 1) {
        if (tid < off) sc_pairs[tid] += sc_pairs[tid + off];
        __syncthreads();
    }
    uint32_t shared_ent = 0;
    if (p.has_shared) {
        shared_ent = (p.tokens + p.tok_per_entry - 1) / p.tok_per_entry;
        for (uint32_t j = tid; j < shared_ent; j += blockDim.x) {
            WorkEntry we;
            we.expert = NVMAI_SLOT_FLAG | 8u;
            we.pair_start = n_pairs + j * p.tok_per_entry;
            we.pair_count = min(p.tok_per_entry, p.tokens - j * p.tok_per_entry);
            we.reserved = 0;
            p.entries[total_ent + j] = we;
        }
        for (uint32_t t = tid; t < p.tokens; t += blockDim.x) {
            p.pair_token[n_pairs + t] = t;
            p.pair_id[n_pairs + t] = n_pairs + t;
        }
    }
    if (tid == 0) {
        p.n_entries[0] = total_ent + shared_ent;
        p.n_entries[1] = sc_pairs[0];
    }
}

// Dense work list: `count` inputs through the expert in slot `slot`.
__global__ void dense_entries_kernel(WorkEntry* entries, uint32_t* n_entries, uint32_t* pair_token,
                                     uint32_t* pair_id, uint32_t count, uint32_t tok_per_entry,
                                     uint32_t slot) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t ents = (count + tok_per_entry - 1) / tok_per_entry;
    if (i < count) { pair_token[i] = i; pair_id[i] = i; }
    if (i < ents) {
        WorkEntry we;
        we.expert = NVMAI_SLOT_FLAG | slot;
        we.pair_start = i * tok_per_entry;
        we.pair_count = min(tok_per_entry, count - i * tok_per_entry);
        we.reserved = 0;
        entries[i] = we;
    }
    if (i == 0) n_entries[0] = ents;
}

// Work list over slots 0..count-1 of one token: entry i -> slot i, output row i,
// input row i (in_is_slot) or 0.
__global__ void slot_entries_kernel(WorkEntry* entries, uint32_t* n_entries, uint32_t* pair_in,
                                    uint32_t* pair_id, uint32_t count, int in_is_slot) {
    const uint32_t i = threadIdx.x;
    if (i < count) {
        WorkEntry we;
        we.expert = NVMAI_SLOT_FLAG | i;
        we.pair_start = i;
        we.pair_count = 1;
        we.reserved = 0;
        entries[i] = we;
        pair_in[i] = in_is_slot ? i : 0u;
        pair_id[i] = i;
    }
    if (i == 0) n_entries[0] = count;
}

// Work list over a subset of the top-k slots of one token (the reference's
// hit/miss split, moe.metal:685-727): slot values >= top_k are skipped.
__global__ void subset_entries_kernel(WorkEntry* entries, uint32_t* n_entries, uint32_t* pair_token,
                                      uint32_t* pair_id, const uint32_t* active_slots,
                                      uint32_t active_count, uint32_t top_k) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    uint32_t n = 0;
    for (uint32_t i = 0; i < active_count; ++i) {
        const uint32_t slot = active_slots[i];
        if (slot >= top_k) continue;
        WorkEntry we;
        we.expert = NVMAI_SLOT_FLAG | slot;
        we.pair_start = n;
        we.pair_count = 1;
        we.reserved = 0;
        entries[n] = we;
        pair_token[n] = 0;
        pair_id[n] = slot;
        ++n;
    }
    n_entries[0] = n;
}

// ---- combine ---------------------------------------------------------------------------
// y[t,d] = base + sum over slots in slot order of w[t,slot] * partial[t*k+slot, d]
// (moe.metal:801-808; CPUExpertFFN.swift:136-138).  base is either a residual in
// the activation type, or the shared expert's partial row scaled by
// 1/(1+exp(-gate_logit)) (utility.metal:61-70), or zero.
struct CombineParams {
    const float* partials;        // [pairs(+tokens), d]
    const uint16_t* w;            // fp16 [tokens, top_k]
    const void* residual;         // optional activations [tokens, res_stride]
    const float* gate_logit;      // optional [tokens]
    int has_shared;               // shared partial rows follow the routed ones
    uint32_t tokens, top_k, d, res_stride, y_stride;
    void* y;
};

template <int ACT>
__global__ __launch_bounds__(256) void combine_kernel(CombineParams p) {
    const uint32_t t = blockIdx.y;
    const uint32_t d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= p.d) return;
    float acc = 0.0f;
    if (p.residual) acc = act_to_f32<ACT>(((const uint16_t*)p.residual)[(size_t)t * p.res_stride + d]);
    if (p.has_shared) {
        float s = p.partials[((size_t)p.tokens * p.top_k + t) * p.d + d];
        if (p.gate_logit) s = __fdiv_rn(s, __fadd_rn(1.0f, expf(-p.gate_logit[t])));
        acc = __fadd_rn(acc, s);
    }
    for (uint32_t r = 0; r < p.top_k; ++r) {
        const float w = f16_to_f32(p.w[(size_t)t * p.top_k + r]);
        acc = __fadd_rn(acc, __fmul_rn(w, p.partials[((size_t)t * p.top_k + r) * p.d + d]));
    }
    ((uint16_t*)p.y)[(size_t)t * p.y_stride + d] = f32_to_act<ACT>(acc);
}

// fp32 [rows, n] -> activations, optionally through act = silu(a) * b of two inputs
template <int ACT>
__global__ void store_act_kernel(const float* a, void* y, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) ((uint16_t*)y)[i] = f32_to_act<ACT>(a[i]);
}

// ---- affine group-64 quantizer ---------------------------------------------------------
// One wave per group of 64 weights: min/max, scale=(max-min)/levels (1 for a
// flat group), both rounded to bf16, then q = clamp(round_half_away((w - b) *
// (1/s)), 0, levels) against the ROUNDED scale and bias (Quantization.swift:59-99,
// :144-175).  Every step is a single IEEE operation so the codes equal the CPU's.
struct QuantParams {
    const void* w;          // [rows, n] fp32 or bf16
    int w_is_bf16;
    uint32_t rows, n, bits;
    uint8_t* packed;
    uint16_t* scales;
    uint16_t* biases;
};

__global__ __launch_bounds__(256) void quantize_affine_kernel(QuantParams p) {
    const uint32_t groups = p.n / NVMAI_GROUP;
    const uint64_t gid = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (gid >= (uint64_t)p.rows * groups) return;
    const int lane = threadIdx.x & 63;
    const uint32_t row = gid / groups, g = gid % groups;
    const size_t e = (size_t)row * p.n + (size_t)g * NVMAI_GROUP + lane;
    const float w = p.w_is_bf16 ? bf16_to_f32(((const uint16_t*)p.w)[e]) : ((const float*)p.w)[e];
    float mn = w, mx = w;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        mn = fminf(mn, shfl_xor_f(mn, off));
        mx = fmaxf(mx, shfl_xor_f(mx, off));
    }
    const float levels = (float)((1u << p.bits) - 1u);
    const float scale_f = (mx == mn) ? 1.0f : __fdiv_rn(__fsub_rn(mx, mn), levels);
    const uint16_t sb = f32_to_bf16(scale_f), bb = f32_to_bf16(mn);
    const float scale = bf16_to_f32(sb), bias = bf16_to_f32(bb);
    const float inv = (scale == 0.0f) ? 0.0f : __fdiv_rn(1.0f, scale);
    float t = roundf(__fmul_rn(__fsub_rn(w, bias), inv));
    t = fminf(fmaxf(t, 0.0f), levels);
    const uint32_t q = (uint32_t)t;
    if (lane == 0) { p.scales[gid] = sb; p.biases[gid] = bb; }
    if (p.bits == 8) {
        p.packed[e] = (uint8_t)q;
    } else {
        const uint32_t hi = shfl_xor_u(q, 1);
        if ((lane & 1) == 0) p.packed[e / 2] = (uint8_t)(q | (hi << 4));
    }
}

// codes -> activations: w = q * scale + bias, two roundings (Quantization.swift:104-119)
template <int ACT>
__global__ void dequantize_affine_kernel(const uint8_t* packed, const uint16_t* scales,
                                         const uint16_t* biases, uint64_t count, uint32_t bits,
                                         uint8_t* codes_out, void* values_out) {
    const uint64_t e = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= count) return;
    uint32_t q;
    if (bits == 8) q = packed[e];
    else { const uint8_t b = packed[e / 2]; q = (e & 1) ? (b >> 4) : (b & 0x0F); }
    if (codes_out) codes_out[e] = (uint8_t)q;
    if (values_out) {
        const float s = bf16_to_f32(scales[e / NVMAI_GROUP]), b = bf16_to_f32(biases[e / NVMAI_GROUP]);
        ((uint16_t*)values_out)[e] = f32_to_act<ACT>(__fadd_rn(__fmul_rn((float)q, s), b));
    }
}

}  // namespace nvmai
