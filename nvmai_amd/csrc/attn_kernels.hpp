// KV-cache quantize-on-write, partial RoPE and GQA decode attention over quantized K/V.
// gfx950, wave64.
#pragma once

#include "common.hpp"

namespace nvmai {

// ---- KV row layout (KVCacheManager.swift:437-446) -----------------------------------------
// row = packed codes (value_bytes, even) | fp16 scales[groups] | fp16 biases[groups]
struct KvFormat {
    uint32_t bits;         // 4, 8 or 16
    uint32_t stride;       // bytes per token row
    uint32_t value_bytes;
    uint32_t elements;     // num_kv_heads * head_dim
};

// ---- quantize on write (kv_cache_quantize.metal:7-73) -------------------------------------
// One wave per (token, group of 64): lane = element.  scale = (max-min)/levels from the
// unrounded fp32 extremes (0 for a flat group), code = round_half_away(clamp((v-bias)/scale)),
// stored scale/bias = fp16 of the fp32 values.  Every step is one IEEE operation.
template <int ACT>
__global__ __launch_bounds__(256) void kv_quantize_kernel(const void* src, uint32_t src_stride, uint8_t* dst,
                                                         KvFormat f, uint32_t tokens) {
    const uint32_t groups = (f.elements + 63) / 64;
    const uint64_t gid = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (gid >= (uint64_t)tokens * groups) return;
    const uint32_t token = gid / groups, g = gid % groups;
    const int lane = threadIdx.x & 63;
    const uint32_t e = g * 64 + lane;
    const bool active = e < f.elements;
    const float v = active ? act_to_f32<ACT>(((const uint16_t*)src)[(size_t)token * src_stride + e]) : 0.0f;
    float mn = active ? v : INFINITY, mx = active ? v : -INFINITY;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        mn = fminf(mn, shfl_xor_f(mn, off));
        mx = fmaxf(mx, shfl_xor_f(mx, off));
    }
    const float levels = f.bits == 4 ? 15.0f : 255.0f;
    const float bias = mn;
    const float scale = mx > mn ? __fdiv_rn(__fsub_rn(mx, mn), levels) : 0.0f;
    uint8_t* row = dst + (size_t)token * f.stride;
    if (lane == 0) {
        reinterpret_cast<uint16_t*>(row + f.value_bytes)[g] = f32_to_f16(scale);
        reinterpret_cast<uint16_t*>(row + f.value_bytes)[groups + g] = f32_to_f16(bias);
    }
    float q = 0.0f;
    if (scale > 0.0f) q = roundf(fminf(fmaxf(__fdiv_rn(__fsub_rn(v, bias), scale), 0.0f), levels));
    const uint32_t code = active ? (uint32_t)q : 0u;
    if (f.bits == 8) {
        if (active) row[e] = (uint8_t)code;
    } else {
        const uint32_t hi = shfl_xor_u(code, 1);     // inactive neighbours contribute 0
        if (active && (lane & 1) == 0) row[e / 2] = (uint8_t)(code | (hi << 4));
    }
}

// The same arithmetic with eight consecutive elements per lane (one 16-byte load) and eight
// lanes per group: for rows of whole groups with 16-byte aligned sources.  min / max do not
// depend on the order of reduction, every other step is per element, so the codes and the fp16
// scale / bias are the same bits as the one-element-per-lane kernel's.
template <int ACT, int BITS>
__global__ __launch_bounds__(256) void kv_quantize_vec_kernel(const void* src, uint32_t src_stride, uint8_t* dst,
                                                             KvFormat f, uint32_t tokens) {
    const uint32_t cpt = f.elements / 8;                          // 16-byte chunks per token
    const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (uint64_t)tokens * cpt) return;                    // whole groups of 8 lanes drop out together
    const uint32_t token = gid / cpt, chunk = gid % cpt;
    const uint4 raw = *reinterpret_cast<const uint4*>((const uint16_t*)src + (size_t)token * src_stride + chunk * 8);
    float v[8];
    act2_to_f32<ACT>(raw.x, v[0], v[1]); act2_to_f32<ACT>(raw.y, v[2], v[3]);
    act2_to_f32<ACT>(raw.z, v[4], v[5]); act2_to_f32<ACT>(raw.w, v[6], v[7]);
    float mn = v[0], mx = v[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) { mn = fminf(mn, v[j]); mx = fmaxf(mx, v[j]); }
#pragma unroll
    for (int off = 4; off >= 1; off >>= 1) {
        mn = fminf(mn, shfl_xor_f(mn, off));
        mx = fmaxf(mx, shfl_xor_f(mx, off));
    }
    constexpr float levels = BITS == 4 ? 15.0f : 255.0f;
    const float bias = mn;
    const float scale = mx > mn ? __fdiv_rn(__fsub_rn(mx, mn), levels) : 0.0f;
    const uint32_t groups = f.elements / 64, g = chunk / 8;
    uint8_t* row = dst + (size_t)token * f.stride;
    if ((chunk & 7u) == 0) {
        reinterpret_cast<uint16_t*>(row + f.value_bytes)[g] = f32_to_f16(scale);
        reinterpret_cast<uint16_t*>(row + f.value_bytes)[groups + g] = f32_to_f16(bias);
    }
    uint32_t code[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float q = 0.0f;
        if (scale > 0.0f) q = roundf(fminf(fmaxf(__fdiv_rn(__fsub_rn(v[j], bias), scale), 0.0f), levels));
        code[j] = (uint32_t)q;
    }
    if (BITS == 8) {
        uint2 o;
        o.x = code[0] | code[1] << 8 | code[2] << 16 | code[3] << 24;
        o.y = code[4] | code[5] << 8 | code[6] << 16 | code[7] << 24;
        *reinterpret_cast<uint2*>(row + chunk * 8) = o;
    } else {
        uint32_t o = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) o |= code[j] << (4 * j);
        *reinterpret_cast<uint32_t*>(row + chunk * 4) = o;
    }
}

// ---- partial RoPE (rope.metal:32-50, 80-102) ------------------------------------------------
// data [tokens, heads, head_dim] in place; pair (i, rot/2 + i), angle = pos * theta^(-2i/rot).
template <int ACT>
__global__ void rope_neox_subdim_kernel(void* data, uint32_t tokens, uint32_t heads, uint32_t head_dim,
                                        uint32_t rotary_dim, const uint32_t* positions, uint32_t position0,
                                        float theta) {
    const uint32_t half_rot = rotary_dim / 2;
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (uint64_t)tokens * heads * half_rot) return;
    const uint32_t pair = i % half_rot;
    const uint64_t th = i / half_rot;              // token * heads + head
    const uint32_t token = th / heads;
    const uint32_t pos = positions ? positions[token] : position0;
    uint16_t* head = (uint16_t*)data + th * head_dim;
    const float exponent = __fdiv_rn(-(float)(2u * pair), (float)rotary_dim);
    const float angle = __fmul_rn((float)pos, powf(theta, exponent));
    const float c = cosf(angle), s = sinf(angle);
    const float x0 = act_to_f32<ACT>(head[pair]), x1 = act_to_f32<ACT>(head[half_rot + pair]);
    head[pair] = f32_to_act<ACT>(__fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s)));
    head[half_rot + pair] = f32_to_act<ACT>(__fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c)));
}

// ---- decode and causal prefill attention -----------------------------------------------------
// "Sequence" b is one query row: a decode step of sequence b, or query token b of a prefill chunk
// (then every b reads the same cache: kv_batch_stride 0).
struct AttnParams {
    const void* q;             // query row of sequence b at q + b * q_stride: [num_q_heads, head_dim]
    const uint8_t* k;          // cache of sequence b at k + b * kv_batch_stride
    const uint8_t* v;
    uint64_t kv_batch_stride;  // bytes
    KvFormat f;
    uint32_t head_dim, num_q_heads, num_kv_heads, batch;
    uint32_t seq_len, kv_start;     // keys [kv_start, seq_len) unless a per-sequence rule below applies;
                                    // seq_len also bounds every row the kernels may touch
    uint32_t num_chunks, chunk_len;
    float scale;
    float* m_part;             // [batch, num_q_heads, num_chunks]
    float* d_part;
    float* o_part;             // [batch, num_q_heads, num_chunks, head_dim]
    void* out;                 // row of sequence b at out + b * out_stride: [num_q_heads, head_dim]
    uint32_t q_stride, out_stride;  // elements
    // per-sequence key ranges: causal (prefill.metal:760-764) or read from device arrays
    uint32_t causal;           // 1: keys [first, min(seq_len, start + b + 1)), first from the window
    uint32_t causal_start, window;
    const uint32_t* seq_lens;  // causal == 0, not null: keys [kv_starts[b] (or kv_start), min(seq_lens[b], seq_len))
    const uint32_t* kv_starts;
    uint32_t ring;             // not 0: row of key p is p % ring (generic kernel only)
    uint32_t cols_q;           // sequences sharing one block of the matrix-core kernel
    uint32_t direct;           // num_chunks == 1: the partial kernel normalises and writes out itself
    // optional output gate (RealForwardRunner.swift:2272-2276, utility.metal:47-58): the combine
    // kernel writes round(out) / (1 + exp(-gate)) -- the rounded row first, as the separate
    // elementwise launch reads it, so the bits are the same.  Row of sequence b at gate + b * gate_stride.
    const uint16_t* gate;
    uint32_t gate_stride;
};

__device__ __forceinline__ void attn_range(const AttnParams& p, uint32_t b, uint32_t& lo, uint32_t& hi) {
    if (p.causal) {
        const uint32_t a = p.causal_start + b + 1u;
        hi = min(p.seq_len, a);
        lo = (p.window != 0u && a > p.window) ? a - p.window : 0u;
    } else {
        hi = p.seq_lens ? min(p.seq_lens[b], p.seq_len) : p.seq_len;
        lo = p.kv_starts ? p.kv_starts[b] : p.kv_start;
    }
    if (lo > hi) lo = hi;
}

__device__ __forceinline__ float kv_load(const uint8_t* row, const KvFormat& f, uint32_t e) {   // attention.metal:89-117
    if (f.bits == 16) return f16_to_f32(reinterpret_cast<const uint16_t*>(row)[e]);
    const uint32_t groups = (f.elements + 63) / 64;
    const uint32_t q = f.bits == 8 ? row[e] : ((e & 1) ? (row[e / 2] >> 4) : (row[e / 2] & 0x0F));
    const uint16_t* meta = reinterpret_cast<const uint16_t*>(row + f.value_bytes);
    return fmaf((float)q, f16_to_f32(meta[e / 64]), f16_to_f32(meta[groups + e / 64]));
}

// Generic split-KV partial (attention.metal:163-261): any head_dim <= 512, any format.
// One block per (sequence, q head, chunk); thread i owns dims i, i+256.
template <int ACT>
__global__ __launch_bounds__(256) void attn_partial_generic_kernel(AttnParams p) {
    __shared__ float red[4];
    const uint32_t chunk = blockIdx.x % p.num_chunks;
    const uint32_t head = (blockIdx.x / p.num_chunks) % p.num_q_heads;
    const uint32_t b = blockIdx.x / (p.num_chunks * p.num_q_heads);
    const uint32_t kvh = head / (p.num_q_heads / p.num_kv_heads);
    uint32_t lo, hi;
    attn_range(p, b, lo, hi);
    const uint32_t p0 = min(lo + chunk * p.chunk_len, hi), p1 = min(p0 + p.chunk_len, hi);
    const uint16_t* qh = (const uint16_t*)p.q + (size_t)b * p.q_stride + (size_t)head * p.head_dim;
    const uint32_t tid = threadIdx.x;
    float qv[2], o[2] = {0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < 2; ++s) qv[s] = tid + 256 * s < p.head_dim ? act_to_f32<ACT>(qh[tid + 256 * s]) : 0.0f;
    float m = -INFINITY, d = 0.0f;
    for (uint32_t pos = p0; pos < p1; ++pos) {
        const uint32_t slot = p.ring ? pos % p.ring : pos;
        const uint8_t* kr = p.k + b * p.kv_batch_stride + (size_t)slot * p.f.stride;
        const uint8_t* vr = p.v + b * p.kv_batch_stride + (size_t)slot * p.f.stride;
        float part = 0.0f;
#pragma unroll
        for (int s = 0; s < 2; ++s)
            if (tid + 256 * s < p.head_dim) part = fmaf(qv[s], kv_load(kr, p.f, kvh * p.head_dim + tid + 256 * s), part);
        part = wave_sum_bcast(part);
        if ((tid & 63) == 0) red[tid >> 6] = part;
        __syncthreads();
        const float sc = (red[0] + red[1] + red[2] + red[3]) * p.scale;
        __syncthreads();
        const float mn = fmaxf(m, sc);
        const float alpha = expf(m - mn), pe = expf(sc - mn);
        d = d * alpha + pe;
#pragma unroll
        for (int s = 0; s < 2; ++s)
            if (tid + 256 * s < p.head_dim)
                o[s] = o[s] * alpha + pe * kv_load(vr, p.f, kvh * p.head_dim + tid + 256 * s);
        m = mn;
    }
    if (p.direct) {                                       // one chunk: no partials, no combine
        uint16_t* orow = (uint16_t*)p.out + (size_t)b * p.out_stride + (size_t)head * p.head_dim;
#pragma unroll
        for (int s = 0; s < 2; ++s)
            if (tid + 256 * s < p.head_dim) orow[tid + 256 * s] = f32_to_act<ACT>(d > 0.0f ? o[s] / d : 0.0f);
        return;
    }
    const size_t base = ((size_t)b * p.num_q_heads + head) * p.num_chunks + chunk;
    if (tid == 0) { p.m_part[base] = m; p.d_part[base] = d; }
#pragma unroll
    for (int s = 0; s < 2; ++s)
        if (tid + 256 * s < p.head_dim) p.o_part[base * p.head_dim + tid + 256 * s] = o[s];
}

// Combine (attention.metal:388-429): m* = max m_c, D = sum d_c e^(m_c - m*),
// out = sum o_c e^(m_c - m*) / D; all chunks empty -> zeros.  Grid (batch * q heads,
// ceil(head_dim / 64)); the four waves of a block split the chunks of 64 output dims.
constexpr uint32_t ATTN_MAX_CHUNKS = 512;

template <int ACT>
__global__ __launch_bounds__(256) void attn_combine_kernel(AttnParams p) {
    __shared__ float wgt[ATTN_MAX_CHUNKS];
    __shared__ float red[8];
    __shared__ float part[4][64];
    const size_t bh = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* mr = p.m_part + bh * p.num_chunks;
    const float* dr = p.d_part + bh * p.num_chunks;
    const float* orow = p.o_part + bh * p.num_chunks * p.head_dim;
    const uint32_t dim = blockIdx.y * 64 + lane;
    uint16_t* out_row = (uint16_t*)p.out + (bh / p.num_q_heads) * p.out_stride + (bh % p.num_q_heads) * p.head_dim;
    const uint16_t* gate_row = p.gate ? p.gate + (bh / p.num_q_heads) * p.gate_stride + (bh % p.num_q_heads) * p.head_dim : nullptr;
    // everything the block reads besides the partial rows is requested at once: a thread's (at most
    // two) chunk maxima and sums, and the gate value of its output element
    uint16_t gate_v = 0;
    if (gate_row && dim < p.head_dim) gate_v = gate_row[dim];
    float mv[2], dv[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
        const uint32_t c = threadIdx.x + 256u * s2, cc = min(c, p.num_chunks - 1u);
        const float m_c = mr[cc], d_c = dr[cc];
        mv[s2] = c < p.num_chunks ? m_c : -INFINITY;
        dv[s2] = c < p.num_chunks ? d_c : 0.0f;
    }
    auto gated = [&](float v) -> uint16_t {
        uint16_t o = f32_to_act<ACT>(v);
        if (gate_row) o = f32_to_act<ACT>(__fdiv_rn(act_to_f32<ACT>(o), __fadd_rn(1.0f, expf(-act_to_f32<ACT>(gate_v)))));
        return o;
    };
    float mloc = fmaxf(fmaxf(-INFINITY, mv[0]), mv[1]);
    mloc = wave_max_f32(mloc);
    if (lane == 0) red[wave] = mloc;
    __syncthreads();
    const float mg = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (mg == -INFINITY) {                                   // uniform over the block
        if (wave == 0 && dim < p.head_dim) out_row[dim] = gated(0.0f);
        return;
    }
    float dloc = 0.0f;
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
        const uint32_t c = threadIdx.x + 256u * s2;
        if (c < p.num_chunks) {
            const float w = expf(mv[s2] - mg);
            wgt[c] = w;
            dloc += dv[s2] * w;
        }
    }
    dloc = wave_sum_bcast(dloc);
    if (lane == 0) red[4 + wave] = dloc;
    __syncthreads();
    const float D = (red[4] + red[5]) + (red[6] + red[7]);
    float acc = 0.0f;
    if (dim < p.head_dim) {
        const float* oc = orow + dim;
#pragma unroll 16
        for (uint32_t c = wave; c < p.num_chunks; c += 4) acc += oc[(size_t)c * p.head_dim] * wgt[c];
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && dim < p.head_dim) {
        const float tot = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
        out_row[dim] = gated(D > 0.0f ? tot / D : 0.0f);
    }
}

// ---- MFMA partial for head_dim 256, 4/8-bit K/V, up to 16 q heads per kv head ---------------
// One block per (batch, kv head, chunk): every q head of the group is served from ONE read of
// the K/V rows.  Each wave walks 32-token steps of the chunk with its own online-softmax state;
// the four waves merge through LDS at the end.
//   S^T[tokens, heads] = K . Q^T   v_mfma_f32_16x16x32_f16, A = the codes themselves, read as
//                                  fp16 subnormals (c * 2^-24: the matrix cores take them
//                                  exactly, and a byte-permute with zero bytes makes two),
//                                  B = q scaled by a power of two per head and cast to fp16;
//                                  one accumulator per 64-wide group so that the row's fp16
//                                  scale and bias are applied exactly:
//                                  s = 2^24 sum_g sc_g acc_g + sum_g bi_g qsum_g
//   O[heads, dims]    = P'_g . V   A = p_t * vsc[t, g] as fp16 (one operand per group),
//                                  B = V codes as fp16 subnormals; O carries the factor 2^-24
//                                  until the wave finishes, the bias goes into a
//                                  per-(head, group) correction.
// Lane roles (l = lane, r = l / 16, i = l % 16):
//   K operand: token i of the 16-token tile, dims 64g + 16r + 8h .. +8 for MFMA call (g, h)
//   Q operand: head i, the same dims
//   S^T accumulators: head i, tokens 4r .. 4r+3 of the tile
//   P' operand: head i, tokens {4r..4r+3 of tile 0, 4r..4r+3 of tile 1} of the 32-token step
//   V operand (group g, tile n): dim 64g + 4i + n, the same eight tokens
//   O accumulators (g, n): dim 64g + 4i + n, heads 4r .. 4r+3
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));

union H8 { h8_t v; uint32_t u[4]; };

__device__ __forceinline__ f4_t mfma16(const H8& a, const H8& b, f4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, c, 0, 0, 0);
}

// s_waitcnt operand: at most n vector-memory loads still in flight, the other counters free.
constexpr int gemm_like_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

// e^x for x <= 0 in two instructions (a multiply and the hardware's 2^x, good to about one ulp; -inf gives
// 0): the library's expf costs a dozen, and the softmax of a step needs nine of them per lane.
__device__ __forceinline__ float attn_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

constexpr int ATTN_HD = 256;
constexpr int ATTN_STEP = 32;

template <int ACT, int BITS>
__global__ __launch_bounds__(256, 2) void attn_partial_mfma_kernel(AttnParams p) {
    // LDS.  Every wave owns a K region and a V region, filled by buffer_load ... lds without
    // touching registers: 32 tokens x the codes of this KV head, the 16-byte chunks of a token
    // XOR-swizzled by the token, then 16 bytes of (scales, biases) per token.  The K region is
    // refilled for the next step as soon as the scores are out, the V region at the end of the
    // step, so each load has half a step to land and one buffer each suffices: 70 KB per block
    // at 8 bits, two blocks per compute unit.  K and V are separate arrays so that the compiler
    // can tell a read of one from a load in flight into the other.  After the loop the K array
    // is the merge area of a two-round tree: [2][16 heads][256 dims] O + [16] m + [16] d.
    // A 64-float scratch per wave serves head-indexed broadcasts.
    constexpr uint32_t CODE_ROW = ATTN_HD * BITS / 8;              // bytes of one token's codes (this head)
    constexpr uint32_t REGION = 32 * CODE_ROW + 512;              // codes | (scales, biases)
    constexpr uint32_t OFF_META = 32 * CODE_ROW;
    constexpr uint32_t MERGE_SLOT = 16 * ATTN_HD + 32;            // floats
    constexpr uint32_t MERGE_BYTES = 2 * MERGE_SLOT * 4;
    constexpr uint32_t KARRAY = 4 * REGION > MERGE_BYTES ? 4 * REGION : MERGE_BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t kst[KARRAY];
    __shared__ __attribute__((aligned(16))) uint8_t vst[4 * REGION];
    __shared__ float bc_all[256];
    // vst is written by load instructions only; a store that never runs keeps the optimizer
    // from treating it as never written (head_dim 0 is rejected by the entry point)
    if (p.head_dim == 0) vst[threadIdx.x] = 0;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, r = lane >> 4;
    float* bc = bc_all + wave * 64;                                // broadcast scratch
    float* merge = reinterpret_cast<float*>(kst);                  // after the loop
    const uint32_t chunk = blockIdx.x % p.num_chunks;
    const uint32_t kvh = (blockIdx.x / p.num_chunks) % p.num_kv_heads;
    const uint32_t n_qb = (p.batch + p.cols_q - 1) / p.cols_q;
    uint32_t qb = blockIdx.x / (p.num_chunks * p.num_kv_heads);
    if (p.causal) qb = n_qb - 1u - qb;                             // the longest key ranges start first
    const uint32_t b = qb * p.cols_q;                              // first sequence of this block
    const uint32_t qpk = p.num_q_heads / p.num_kv_heads;           // <= 16
    // Column i of the score tile is (sequence b + i / qpk, q head i % qpk of this kv head): a decode
    // step has cols_q = 1, a prefill chunk packs 16 / qpk query tokens into the sixteen columns.
    const uint32_t cols = min(p.cols_q, p.batch - b) * qpk;        // live columns
    const bool live = (uint32_t)i < cols;
    const uint32_t my_b = b + (live ? (uint32_t)i / qpk : 0u), my_h = kvh * qpk + (live ? (uint32_t)i % qpk : 0u);
    uint32_t lo_i, hi_i;                                           // key range of this lane's column
    attn_range(p, my_b, lo_i, hi_i);
    uint32_t blo = live ? lo_i : 0xFFFFFFFFu, bhi = live ? hi_i : 0u;
    if (!live) lo_i = hi_i = 0u;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        blo = min(blo, shfl_xor_u(blo, off));
        bhi = max(bhi, shfl_xor_u(bhi, off));
    }
    blo = __builtin_amdgcn_readfirstlane(blo);                     // the union of the block's ranges
    bhi = __builtin_amdgcn_readfirstlane(bhi);
    const uint32_t p0 = min(blo + chunk * p.chunk_len, bhi), p1 = min(p0 + p.chunk_len, bhi);
    const uint32_t groups_total = (p.f.elements + 63) / 64;
    const uint32_t code_off = kvh * ATTN_HD * BITS / 8;            // this head's codes inside a row
    const uint32_t meta_sc = p.f.value_bytes + 2 * (kvh * 4);      // 4 fp16 scales of this head
    const uint32_t meta_bi = p.f.value_bytes + 2 * groups_total + 2 * (kvh * 4);
    const uint8_t* kbase = p.k + b * p.kv_batch_stride;
    const uint8_t* vbase = p.v + b * p.kv_batch_stride;

    // ---- Q: head i (zero for i >= qpk), scaled to fp16; operands and per-group sums
    H8 qop[4][2];
    float qsum[4];
    float q_unscale;                                               // scale * 2^-k of head i
    {
        const uint16_t* qh = (const uint16_t*)p.q + (size_t)my_b * p.q_stride + (size_t)my_h * ATTN_HD;
        float qf[4][2][8];
        float amax = 0.0f;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint4 raw = *reinterpret_cast<const uint4*>(qh + 64 * g + 16 * r + 8 * h);
                act2_to_f32<ACT>(raw.x, qf[g][h][0], qf[g][h][1]); act2_to_f32<ACT>(raw.y, qf[g][h][2], qf[g][h][3]);
                act2_to_f32<ACT>(raw.z, qf[g][h][4], qf[g][h][5]); act2_to_f32<ACT>(raw.w, qf[g][h][6], qf[g][h][7]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (!live) qf[g][h][e] = 0.0f;
                    amax = fmaxf(amax, fabsf(qf[g][h][e]));
                }
            }
        amax = fmaxf(amax, shfl_xor_f(amax, 16));
        amax = fmaxf(amax, shfl_xor_f(amax, 32));
        // power of two mapping amax into [1024, 2048) (1 for zero / non-finite rows)
        const uint32_t ex = (__float_as_uint(amax) >> 23) & 0xFFu;
        float sc = 1.0f, isc = 1.0f;
        if (ex >= 24u && ex <= 254u) { sc = __uint_as_float((264u - ex) << 23); isc = __uint_as_float((ex - 10u) << 23); }
        q_unscale = p.scale * isc;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float s = 0.0f;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                uint16_t hb[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    // 4 bit: the K codes of elements 1, 3, 5, 7 are used where they lie, at bits 4..7 of a half
                    // (16 c * 2^-24, see the operand build in the loop), so those query elements carry 1/16
                    const bool sixteenth = BITS == 4 && (e & 1);
                    hb[e] = f32_to_f16(qf[g][h][e] * (sixteenth ? sc * 0.0625f : sc));
                    s += f16_to_f32(hb[e]) * (sixteenth ? 16.0f : 1.0f);
                }
                if (BITS == 8) {
                    // K codes unpack in natural byte order: pairs (0,1) (2,3) (4,5) (6,7)
#pragma unroll
                    for (int w = 0; w < 4; ++w) qop[g][h].u[w] = hb[2 * w] | ((uint32_t)hb[2 * w + 1] << 16);
                } else {
                    // 4-bit codes unpack as pairs (j, j+4) of the dword's eight nibbles
#pragma unroll
                    for (int w = 0; w < 4; ++w) qop[g][h].u[w] = hb[w] | ((uint32_t)hb[w + 4] << 16);
                }
            }
            s += shfl_xor_f(s, 16);
            s += shfl_xor_f(s, 32);
            qsum[g] = s;                                           // over all 64 dims of group g, head i
        }
    }

    f4_t oacc[4][4];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int n = 0; n < 4; ++n) oacc[g][n] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, d_run = 0.0f;                          // head i; d over this lane's tokens only
    float corr[4] = {0.0f, 0.0f, 0.0f, 0.0f};                       // head i, this lane's tokens only

    auto slot_tok = [&](int t) { return (uint32_t)((t >> 2) * 16 + 4 * r + (t & 3)); };   // token of slot t inside the step
    // Buffer loads: a scalar resource per cache, 32-bit offsets; reads past the end of the
    // sequence's rows return zero instead of faulting (tokens past the chunk are masked anyway).
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(kbase), 0, (int)(p.seq_len * p.f.stride), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(vbase), 0, (int)(p.seq_len * p.f.stride), 0x00020000);
    // One load instruction moves 1 KB = the codes of 4 (8 bit) or 8 (4 bit) tokens: lane l takes
    // chunk (l % LPT) ^ token of token l / LPT, which lands in slot l % LPT of that token.
    constexpr int LPT = CODE_ROW / 16;                              // lanes (16-byte chunks) per token
    constexpr int TPI = 64 / LPT;                                   // tokens per instruction
    const uint32_t d_tok = lane / LPT, d_slot = lane % LPT;
    // The 16-byte chunks of a token are XOR-swizzled so that the operand reads below touch every bank once.
    // 8 bit (256-byte rows, sixteen chunks): chunk ^ token.  4 bit (128-byte rows: the token's lowest bit already
    // picks the half of the 256 bytes the banks span, and only eight chunks): chunk ^ (token >> 1) -- swizzled by
    // the token's low three bits, tokens 8 apart fell on the same banks (two-way conflicts in both operand reads).
    const uint32_t d_chunk16 = BITS == 8 ? ((d_slot ^ d_tok) & (LPT - 1)) * 16u        // ^ 64 (j & 3) per instruction
                                         : ((d_slot ^ (d_tok >> 1)) & (LPT - 1)) * 16u;  // ^ 64 (j & 1) per instruction
    const uint32_t m_part = (lane & 3) < 2 ? meta_sc + 4 * (lane & 3) : meta_bi + 4 * ((lane & 3) - 2);
    uint8_t* const myk = kst + wave * REGION;
    uint8_t* const myv = vst + wave * REGION;
    constexpr int N_LOADS = 32 / TPI + 2;                           // load instructions of one region
    auto issue_region = [&](uint32_t s0, const __amdgpu_buffer_rsrc_t& rs, uint8_t* st) {
        const uint32_t row = (s0 + d_tok) * p.f.stride;
#pragma unroll
        for (int j = 0; j < 32 / TPI; ++j) {
            const uint32_t voff = row + (d_chunk16 ^ (64u * (j & (BITS == 8 ? 3 : 1))));
            const uint32_t soff = (uint32_t)(j * TPI) * p.f.stride + code_off;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(st + j * 1024), 16, voff, soff, 0, 0);
        }
        const uint32_t mrow = (s0 + (lane >> 2)) * p.f.stride + m_part;
#pragma unroll
        for (int m = 0; m < 2; ++m)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(st + OFF_META + m * 256), 4, mrow,
                                                     (uint32_t)(16 * m) * p.f.stride, 0, 0);
    };
    // (requested after the query loads: loads return in order, and the queries' preparation then
    // overlaps the flight of the rows -- the other order was measured 0.7 us slower per launch)
    const uint32_t s_first = p0 + wave * ATTN_STEP;
    if (s_first < p1) { issue_region(s_first, krsrc, myk); issue_region(s_first, vrsrc, myv); }

    for (uint32_t s0 = s_first; s0 < p1; s0 += 4 * ATTN_STEP) {
        const bool more = s0 + 4 * ATTN_STEP < p1;                  // wave-uniform
        // the K region of this step has landed; only this step's V loads may still be in flight
        __builtin_amdgcn_s_waitcnt(gemm_like_vmcnt(N_LOADS));
        bool tok_ok[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t pos = s0 + slot_tok(t);
            tok_ok[t] = pos < p1 && pos >= lo_i && pos < hi_i;
        }

        // ---- S^T = K . Q^T per group, then the exact affine correction
        float sv[8];                                                // scores of head i at this lane's 8 tokens
#pragma unroll
        for (int tile = 0; tile < 2; ++tile) {
            // the scales and biases of this lane's four tokens of the tile, requested ahead of the products: read
            // where they are used, each read was waited for on the spot, inside a branch of its own
            uint4 km4[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) km4[t] = *reinterpret_cast<const uint4*>(myk + OFF_META + slot_tok(tile * 4 + t) * 16);
            f4_t sacc[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                sacc[g] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
                // codes of token i of the tile, dims 64 g + 16 r .. +16
                uint32_t kw[4];
                if (BITS == 8) {
                    const uint4 w = *reinterpret_cast<const uint4*>(myk + (tile * 16 + i) * CODE_ROW + (((4 * g + r) ^ i) & 15) * 16);
                    kw[0] = w.x; kw[1] = w.y; kw[2] = w.z; kw[3] = w.w;
                } else {
                    const uint2 w = *reinterpret_cast<const uint2*>(myk + (tile * 16 + i) * CODE_ROW + (((2 * g + (r >> 1)) ^ (i >> 1)) & 7) * 16 + (r & 1) * 8);
                    kw[0] = w.x; kw[1] = w.y;
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    H8 a;
                    if (BITS == 8) {
                        const uint32_t w0 = kw[2 * h], w1 = kw[2 * h + 1];
                        a.u[0] = __builtin_amdgcn_perm(w0, w0, 0x0C050C04u);      // [c0, 0, c1, 0]
                        a.u[1] = __builtin_amdgcn_perm(w0, w0, 0x0C070C06u);
                        a.u[2] = __builtin_amdgcn_perm(w1, w1, 0x0C050C04u);
                        a.u[3] = __builtin_amdgcn_perm(w1, w1, 0x0C070C06u);
                    } else {
                        // pairs (j, j + 4) of the dword's nibbles; a nibble at bits 4..7 of a half reads as 16 c * 2^-24
                        // (still a subnormal), which the query's 1/16 takes back: one shift instead of three
                        const uint32_t w = kw[h], w8 = w >> 8;
                        a.u[0] = w & 0x000F000Fu; a.u[1] = w & 0x00F000F0u;
                        a.u[2] = w8 & 0x000F000Fu; a.u[3] = w8 & 0x00F000F0u;
                    }
                    sacc[g] = mfma16(a, qop[g][h], sacc[g]);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int slot = tile * 4 + t;
                const uint4 km = km4[t];
                // the fp16 scales and biases go into the multiply-adds as they are (mixed-precision fma reads either
                // half of a dword): extracted and converted on their own they cost two more instructions each
                typedef _Float16 hh2_t __attribute__((ext_vector_type(2)));
                const hh2_t s01 = __builtin_bit_cast(hh2_t, km.x), s23 = __builtin_bit_cast(hh2_t, km.y);
                const hh2_t b01 = __builtin_bit_cast(hh2_t, km.z), b23 = __builtin_bit_cast(hh2_t, km.w);
                float acc_s = __builtin_fmaf((float)s01.x, sacc[0][t], 0.0f);
                acc_s = __builtin_fmaf((float)s01.y, sacc[1][t], acc_s);
                acc_s = __builtin_fmaf((float)s23.x, sacc[2][t], acc_s);
                acc_s = __builtin_fmaf((float)s23.y, sacc[3][t], acc_s);
                float acc_b = __builtin_fmaf((float)b01.x, qsum[0], 0.0f);
                acc_b = __builtin_fmaf((float)b01.y, qsum[1], acc_b);
                acc_b = __builtin_fmaf((float)b23.x, qsum[2], acc_b);
                acc_b = __builtin_fmaf((float)b23.y, qsum[3], acc_b);
                float val = fmaf(acc_s, 16777216.0f, acc_b) * q_unscale;
#if defined(__HIP_DEVICE_COMPILE__)
                asm("" : "+v"(val));                        // computed for every slot, masked by a select: no branch per slot
#endif
                sv[slot] = tok_ok[slot] ? val : -INFINITY;
            }
        }

        // the scores are out: the K region takes the next step's rows (every read of it has
        // returned, the score arithmetic used them)
        __builtin_amdgcn_s_waitcnt(0xC07F);                         // lgkmcnt(0)
        if (more) issue_region(s0 + 4 * ATTN_STEP, krsrc, myk);

        // ---- online softmax for head i (its tokens are spread over the four lane quarters)
        float mx = sv[0];
#pragma unroll
        for (int t = 1; t < 8; ++t) mx = fmaxf(mx, sv[t]);
        mx = fmaxf(mx, shfl_xor_f(mx, 16));
        mx = fmaxf(mx, shfl_xor_f(mx, 32));
        const float m_new = fmaxf(m_run, mx);                       // -inf while the column has seen no key yet
        const bool none = m_new == -INFINITY;
        const float alpha = none ? 1.0f : attn_exp(m_run - m_new);
        float pe[8], psum = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) { pe[t] = none ? 0.0f : attn_exp(sv[t] - m_new); psum += pe[t]; }
        d_run = d_run * alpha + psum;
        m_run = m_new;

        // ---- P'_g = p * vsc_g as fp16; correction terms; rescale O by alpha of its heads
        // the V region of this step has landed; the K loads just issued may still be in flight
        if (more) __builtin_amdgcn_s_waitcnt(gemm_like_vmcnt(N_LOADS)); else __builtin_amdgcn_s_waitcnt(0x0F70);
        uint4 vm[8];                                                // (sc.x, sc.y, bi.x, bi.y) of the 8 token slots
#pragma unroll
        for (int t = 0; t < 8; ++t) vm[t] = *reinterpret_cast<const uint4*>(myv + OFF_META + slot_tok(t) * 16);
        // Both factors of p * vsc are fp16 values (the cache stores fp16 scales and biases, p <= 1 is rounded to
        // fp16 once), so two tokens take one packed multiply, and the bias correction one two-term dot product:
        // per group four byte-permutes pick the (token 2w, token 2w + 1) pair of scales and of biases.
        typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
        typedef float f2_t __attribute__((ext_vector_type(2)));
        H8 pop[4];
        h2_t p2[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) p2[w] = __builtin_convertvector(f2_t{pe[2 * w], pe[2 * w + 1]}, h2_t);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float c = corr[g] * alpha;
            const uint32_t sel = (g & 1) ? 0x07060302u : 0x05040100u;   // the group's half of (token 2w, token 2w + 1)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t sc2 = __builtin_amdgcn_perm(g < 2 ? vm[2 * w + 1].x : vm[2 * w + 1].y, g < 2 ? vm[2 * w].x : vm[2 * w].y, sel);
                const uint32_t bi2 = __builtin_amdgcn_perm(g < 2 ? vm[2 * w + 1].z : vm[2 * w + 1].w, g < 2 ? vm[2 * w].z : vm[2 * w].w, sel);
                pop[g].u[w] = __builtin_bit_cast(uint32_t, p2[w] * __builtin_bit_cast(h2_t, sc2));
                c = __builtin_amdgcn_fdot2(p2[w], __builtin_bit_cast(h2_t, bi2), c, false);
            }
            corr[g] = c;
        }
        if (i < 16 && r == 0) bc[i] = alpha;                        // head-indexed broadcast through LDS
        __builtin_amdgcn_wave_barrier();
        const float4 al = *reinterpret_cast<const float4*>(bc + 4 * r);
        __builtin_amdgcn_wave_barrier();
        if (__any(alpha != 1.0f)) {                                 // a running maximum moved somewhere in the wave
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int n = 0; n < 4; ++n) {
                    oacc[g][n][0] *= al.x; oacc[g][n][1] *= al.y; oacc[g][n][2] *= al.z; oacc[g][n][3] *= al.w;
                }
        }

        // ---- O += P'_g . V   (B operand: dim 64g + 4i + n, this lane's 8 tokens)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            // this lane's 4 dims (64 g + 4 i ..) of its 8 token slots
            uint32_t vr[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const uint32_t tk = slot_tok(t);
                if (BITS == 8) vr[t] = *reinterpret_cast<const uint32_t*>(myv + tk * CODE_ROW + (((4 * g + (i >> 2)) ^ tk) & 15) * 16 + (i & 3) * 4);
                else vr[t] = *reinterpret_cast<const uint16_t*>(myv + tk * CODE_ROW + (((2 * g + (i >> 3)) ^ (tk >> 1)) & 7) * 16 + (i & 7) * 2);
            }
            uint32_t pair4[4];                                      // 4-bit: nibbles of two tokens side by side
            if (BITS == 4) {
#pragma unroll
                for (int w = 0; w < 4; ++w) pair4[w] = __builtin_amdgcn_perm(vr[2 * w + 1], vr[2 * w], 0x05040100u);
            }
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                H8 bop;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if (BITS == 8) {
                        // byte n of two token dwords -> [a.n, 0, c2.n, 0]: two fp16 subnormals
                        const uint32_t sel = 0x0C000C00u | (uint32_t)n | ((uint32_t)(4 + n) << 16);
                        bop.u[w] = __builtin_amdgcn_perm(vr[2 * w + 1], vr[2 * w], sel);
                    } else {
                        // dims n = 1, 3 where they lie (bits 4..7 of a half: 16 c * 2^-24, taken back when O leaves its scale)
                        bop.u[w] = ((n & 2) ? pair4[w] >> 8 : pair4[w]) & ((n & 1) ? 0x00F000F0u : 0x000F000Fu);
                    }
                }
                oacc[g][n] = mfma16(pop[g], bop, oacc[g][n]);
            }
        }
        // every read of the V region has returned (the MFMAs took them): it takes the next step's rows
        __builtin_amdgcn_s_waitcnt(0xC07F);
        if (more) issue_region(s0 + 4 * ATTN_STEP, vrsrc, myv);
    }

    // ---- finish this wave: d and corr over the four quarters, corr folded into O
    d_run += shfl_xor_f(d_run, 16);
    d_run += shfl_xor_f(d_run, 32);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        corr[g] += shfl_xor_f(corr[g], 16);
        corr[g] += shfl_xor_f(corr[g], 32);
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        if (r == 0) bc[i] = corr[g];
        __builtin_amdgcn_wave_barrier();
        const float4 cg = *reinterpret_cast<const float4*>(bc + 4 * r);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int n = 0; n < 4; ++n) {                               // O leaves its 2^-24 here
            const float unscale = (BITS == 4 && (n & 1)) ? 1048576.0f : 16777216.0f;   // 4 bit, odd dims: 2^24 / 16
            oacc[g][n][0] = fmaf(oacc[g][n][0], unscale, cg.x); oacc[g][n][1] = fmaf(oacc[g][n][1], unscale, cg.y);
            oacc[g][n][2] = fmaf(oacc[g][n][2], unscale, cg.z); oacc[g][n][3] = fmaf(oacc[g][n][3], unscale, cg.w);
        }
    }

    // ---- merge the four waves, attention.metal:388-429's rule, as a tree of pairwise merges
    // (3 -> 2 and 1 -> 0, then 2 -> 0).  The merge area lies over the K array: every wave must be
    // through with its loop first.
    auto put_state = [&](float* slot) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int t = 0; t < 4; ++t) slot[(4 * r + t) * ATTN_HD + 64 * g + 4 * i + n] = oacc[g][n][t];
        if (r == 0) { slot[16 * ATTN_HD + i] = m_run; slot[16 * ATTN_HD + 16 + i] = d_run; }
    };
    auto take_state = [&](const float* slot) {
        const float m_o = slot[16 * ATTN_HD + i], d_o = slot[16 * ATTN_HD + 16 + i];
        const float m_new = fmaxf(m_run, m_o);
        const float wa = m_run == -INFINITY ? 0.0f : expf(m_run - m_new);
        const float wb = m_o == -INFINITY ? 0.0f : expf(m_o - m_new);
        d_run = d_run * wa + d_o * wb;
        m_run = m_new;
        // weights of heads 4r .. 4r+3 (the O layout) through the broadcast scratch
        if (r == 0) bc[i] = wa;
        __builtin_amdgcn_wave_barrier();
        const float4 a4 = *reinterpret_cast<const float4*>(bc + 4 * r);
        __builtin_amdgcn_wave_barrier();
        if (r == 0) bc[i] = wb;
        __builtin_amdgcn_wave_barrier();
        const float4 b4 = *reinterpret_cast<const float4*>(bc + 4 * r);
        __builtin_amdgcn_wave_barrier();
        const float wa4[4] = {a4.x, a4.y, a4.z, a4.w}, wb4[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    oacc[g][n][t] = oacc[g][n][t] * wa4[t] + slot[(4 * r + t) * ATTN_HD + 64 * g + 4 * i + n] * wb4[t];
    };
    __syncthreads();
    if (wave & 1) put_state(merge + (wave >> 1) * MERGE_SLOT);
    __syncthreads();
    if (!(wave & 1)) take_state(merge + (wave >> 1) * MERGE_SLOT);
    __syncthreads();
    if (wave == 2) put_state(merge);
    __syncthreads();
    if (wave != 0) return;
    take_state(merge);
    // column c -> (sequence b + c / qpk, q head kvh * qpk + c % qpk)
    if (p.direct) {                                                 // one chunk: normalise and write the rows
        if (r == 0) bc[i] = d_run;
        __builtin_amdgcn_wave_barrier();
        const float4 d4 = *reinterpret_cast<const float4*>(bc + 4 * r);
        __builtin_amdgcn_wave_barrier();
        const float dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t c = 4 * r + t;
            if (c >= cols) continue;
            uint16_t* dst = (uint16_t*)p.out + (size_t)(b + c / qpk) * p.out_stride + (size_t)(kvh * qpk + c % qpk) * ATTN_HD;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 o2;
                o2.x = f32_to_act<ACT>(dd[t] > 0.0f ? oacc[g][0][t] / dd[t] : 0.0f) |
                       ((uint32_t)f32_to_act<ACT>(dd[t] > 0.0f ? oacc[g][1][t] / dd[t] : 0.0f) << 16);
                o2.y = f32_to_act<ACT>(dd[t] > 0.0f ? oacc[g][2][t] / dd[t] : 0.0f) |
                       ((uint32_t)f32_to_act<ACT>(dd[t] > 0.0f ? oacc[g][3][t] / dd[t] : 0.0f) << 16);
                *reinterpret_cast<uint2*>(dst + 64 * g + 4 * i) = o2;
            }
        }
        return;
    }
    if (r == 0 && live) {
        const size_t at = ((size_t)my_b * p.num_q_heads + my_h) * p.num_chunks + chunk;
        p.m_part[at] = m_run;
        p.d_part[at] = d_run;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t c = 4 * r + t;
        if (c >= cols) continue;
        float* dst = p.o_part + (((size_t)(b + c / qpk) * p.num_q_heads + kvh * qpk + c % qpk) * p.num_chunks + chunk) * ATTN_HD;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 o4 = {oacc[g][0][t], oacc[g][1][t], oacc[g][2][t], oacc[g][3][t]};
            *reinterpret_cast<float4*>(dst + 64 * g + 4 * i) = o4;
        }
    }
}

}  // namespace nvmai
