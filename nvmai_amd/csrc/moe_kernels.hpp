// Decode-side kernels of the quantized MoE path: affine-row GEMV engines
// (gate/up SwiGLU and down), router logits, device top-k + expert work list,
// weighted combine, and the affine group-64 quantizer.  gfx950, wave64.
#pragma once

#include "common.hpp"

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
    // dense launches (one matrix against dense_count input rows, no work list in memory):
    uint32_t dense_count;
    void* out_act;               // optional 16-bit copy of the result, rows out_act_stride apart;
    uint32_t out_act_stride;     // `out` may then be null
    // dense launches with the PRENORM body: x holds the residual stream's rows and the inputs are
    // rmsnorm(round(x + pre_delta)) * pre_weight, made by every block for itself (stage_prenorm_rows);
    // block 0 stores the updated residual rows to pre_hidden_out.  n <= 2048, rows 16-byte aligned.
    const uint16_t* pre_delta;
    const uint16_t* pre_weight;
    uint16_t* pre_hidden_out;
    uint16_t* pre_normed_out;    // optional: block 0 also stores the normed rows
    uint32_t pre_delta_stride, pre_hidden_stride, pre_normed_stride;
    float pre_eps;
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

// ---- residual add + RMSNorm as the prologue of a kernel that stages its input rows in LDS ----------
// Rows t0 .. t0 + nt - 1 of x (the residual stream) are summed with their delta rows, rounded,
// normed and left in xl [nt][d] as 16-bit activations: the arithmetic and the summation order of
// residual_add_rmsnorm / rms_direct_kernel, so the same bits.  The `writer` block also stores the
// updated residual rows to hidden_out (never x itself: other blocks still read it) and, when asked, the
// normed rows to normed_out.
// raw: d 16-bit values of LDS.  A thread keeps its 16-byte pieces of the row in registers between
// the add and the scaling (d <= 8192), every load is issued before the first use, and every wave
// sums the squares for itself (the same 64-lane order, so the same bits) -- no broadcast, one
// barrier less.  Ends with a barrier.
struct PreNormArgs {
    const uint16_t* x;             // [rows, x_stride] residual stream
    uint32_t x_stride;
    const uint16_t* delta;         // [rows, delta_stride] or null (norm only)
    uint32_t delta_stride;
    const uint16_t* weight;        // BF16 [d]
    uint16_t* hidden_out;          // [rows, hidden_stride] or null
    uint32_t hidden_stride;
    uint16_t* normed_out;          // [rows, normed_stride] or null
    uint32_t normed_stride;
    float eps;
    uint32_t d;
};
constexpr int ROUTER_PRE_PIECES = 4;                 // 16-byte pieces per thread: d <= 8192

template <int ACT>
__device__ __forceinline__ void stage_prenorm_rows(const PreNormArgs& p, uint32_t t0, uint32_t nt, uint16_t* xl,
                                                   uint16_t* raw, const bool writer) {
    const uint32_t per_row = p.d / 8, lane = threadIdx.x & 63;
    for (uint32_t t = 0; t < nt; ++t) {
        const uint16_t* h = p.x + (size_t)(t0 + t) * p.x_stride;
        uint4 v[ROUTER_PRE_PIECES], dl[ROUTER_PRE_PIECES], w[ROUTER_PRE_PIECES];
#pragma unroll
        for (int k = 0; k < ROUTER_PRE_PIECES; ++k) {
            const uint32_t c = threadIdx.x + 256 * k;
            if (c >= per_row) break;
            v[k] = *reinterpret_cast<const uint4*>(h + c * 8);
            if (p.delta) dl[k] = *reinterpret_cast<const uint4*>(p.delta + (size_t)(t0 + t) * p.delta_stride + c * 8);
            w[k] = *reinterpret_cast<const uint4*>(p.weight + c * 8);
        }
#pragma unroll
        for (int k = 0; k < ROUTER_PRE_PIECES; ++k) {
            const uint32_t c = threadIdx.x + 256 * k;
            if (c >= per_row) break;
            if (p.delta) {
                uint32_t* vv = reinterpret_cast<uint32_t*>(&v[k]);
                const uint32_t* dd = reinterpret_cast<const uint32_t*>(&dl[k]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float a0, a1, b0, b1;
                    act2_to_f32<ACT>(vv[j], a0, a1);
                    act2_to_f32<ACT>(dd[j], b0, b1);
                    vv[j] = (uint32_t)f32_to_act<ACT>(__fadd_rn(a0, b0)) | ((uint32_t)f32_to_act<ACT>(__fadd_rn(a1, b1)) << 16);
                }
            }
            reinterpret_cast<uint4*>(raw)[c] = v[k];
            if (writer && p.hidden_out)
                *reinterpret_cast<uint4*>(p.hidden_out + (size_t)(t0 + t) * p.hidden_stride + c * 8) = v[k];
        }
        __syncthreads();
        // the stated order: lane l over the elements l, l + 64, ...; eight reads in flight at a time
        float acc = 0.0f;
        for (uint32_t i0 = lane; i0 < p.d; i0 += 512) {
            uint16_t e[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) e[j] = i0 + 64 * j < p.d ? raw[i0 + 64 * j] : (uint16_t)0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (i0 + 64 * j >= p.d) break;
                const float x = act_to_f32<ACT>(e[j]);
                acc = fmaf(x, x, acc);
            }
        }
        const float inv = rms_inverse(rms_wave_sum(acc), p.d, p.eps);
#pragma unroll
        for (int k = 0; k < ROUTER_PRE_PIECES; ++k) {
            const uint32_t c = threadIdx.x + 256 * k;
            if (c >= per_row) break;
            const uint32_t* vv = reinterpret_cast<const uint32_t*>(&v[k]);
            const uint32_t* ww = reinterpret_cast<const uint32_t*>(&w[k]);
            uint4 o;
            uint32_t* oo = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float a0, a1, w0, w1;
                act2_to_f32<ACT>(vv[j], a0, a1);
                act2_to_f32<ACT_BF16>(ww[j], w0, w1);
                oo[j] = (uint32_t)f32_to_act<ACT>(__fmul_rn(__fmul_rn(a0, inv), w0)) |
                        ((uint32_t)f32_to_act<ACT>(__fmul_rn(__fmul_rn(a1, inv), w1)) << 16);
            }
            reinterpret_cast<uint4*>(xl)[t * per_row + c] = o;
            if (writer && p.normed_out)
                *reinterpret_cast<uint4*>(p.normed_out + (size_t)(t0 + t) * p.normed_stride + c * 8) = o;
        }
        __syncthreads();                             // xl is complete; raw is rewritten by the next row
    }
}

// Offset, in the fast engine's dynamic LDS, of the area behind its own arrays (16-byte aligned).
__host__ __device__ inline size_t rows_fast_lds_base(uint32_t n, int nch, int seg) {
    const size_t own = (size_t)4 /* MAX_TOK */ * (n / 8) * 16 + (size_t)4 * nch * seg * 8 + 4 * 4 * 4 + 4 * 4;
    return (own + 15) & ~(size_t)15;
}

// ---- fast engine ------------------------------------------------------------
// A row of n codes is n*BITS/128 chunks of 16 bytes.  SEG lanes share a row
// (SEG*NCH chunks), so one wave covers 64/SEG rows per load instruction and
// every load instruction moves 1 KiB of contiguous weights.  A block owns a run
// of rows of one work entry; weight loads are double-buffered in registers, the
// first batch being issued before the inputs are staged.
//
// Arithmetic.  The kernel is fed by HBM only if the VALU work per weight byte is
// small, so the inner product runs on v_dot2_f32_f16 (two multiply-adds per lane
// per instruction, fp32 accumulate):
//   - a code q becomes the fp16 value 1024 + q by OR-ing it under the constant
//     0x6400 (exact: fp16 has a unit ulp in [1024, 2048)); one byte-permute or
//     and-or instruction builds two such values;
//   - each input row is scaled by a power of two so that its largest magnitude
//     lies in [1024, 2048) and is converted to fp16.  For 16-bit activations the
//     conversion is exact for everything within 2^-24 of the row maximum, i.e.
//     to fp32 precision; fp32 inputs (the SwiGLU activations entering the down
//     projection) are rounded to 11 significant bits, as the reference rounds
//     them to fp16 in memory (moe.metal:682);
//   - per chunk sum(q*x) = dot2-sum - 1024*sum(x), then the reference's factoring
//     (nvmai_kernels.h:19-21): acc += scale * sum(q*x) + bias * sum(x), with
//     sum(x) hoisted out of the row loop as int4_affine_gemv.c:41-53 does;
//   - the row result is multiplied by the inverse power of two.
template <int BITS, int SEG, int NCH, bool DUAL, int RPI>
struct RowStage {
    uint4 qa[RPI][NCH], qb[DUAL ? RPI : 1][NCH];
    uint16_t sa[RPI][NCH], ba[RPI][NCH], sb[DUAL ? RPI : 1][NCH], bb[DUAL ? RPI : 1][NCH];
};

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
}

// 16 bytes of codes -> packed fp16 pairs.  8 bit: pair m holds the elements (2m, 2m+1) as
// 1024 + q.  4 bit: dword d of the chunk yields pairs 4d+j holding the elements (8d+j, 8d+j+4);
// the staged inputs are packed the same way.  A nibble at bits 0..3 of a half becomes 1024 + q
// under 0x6400, a nibble at bits 4..7 becomes 64 + q under 0x5400 (the binade whose fourth
// mantissa bit weighs one), so the odd pairs need no shift of their own: one shift by 8 and four
// and-or instructions per dword.  The odd pairs' offset of 64 instead of 1024 is taken back with
// the sum of the inputs at their positions (ODD_PAIR_OFFSET_GAP).
constexpr float ODD_PAIR_OFFSET_GAP = 1024.0f - 64.0f;
// The 4-bit masks and exponent patterns arrive in registers (NibbleConsts, made opaque to the
// compiler once per kernel): written as literals every AND-OR splits into a v_and and a v_or,
// because the three-operand v_and_or_b32 takes no literal on this target; with the mask in a
// scalar and the pattern in a vector register it is one instruction.
struct NibbleConsts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};
__device__ __forceinline__ NibbleConsts nibble_consts() {
    NibbleConsts c{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
#if defined(__HIP_DEVICE_COMPILE__)
    asm("" : "+s"(c.mask_lo));
    asm("" : "+s"(c.mask_hi));
    asm("" : "+v"(c.magic_lo));
    asm("" : "+v"(c.magic_hi));
#endif
    return c;
}

template <int BITS>
__device__ __forceinline__ void unpack_pairs(const uint4& w, uint32_t* qp, const NibbleConsts& nc) {
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        if (BITS == 8) {
            qp[2 * d] = __builtin_amdgcn_perm(ws[d], 0x64646464u, 0x00050004u);
            qp[2 * d + 1] = __builtin_amdgcn_perm(ws[d], 0x64646464u, 0x00070006u);
        } else {
            const uint32_t hi = ws[d] >> 8;
            qp[4 * d] = (ws[d] & nc.mask_lo) | nc.magic_lo;
            qp[4 * d + 1] = (ws[d] & nc.mask_hi) | nc.magic_hi;
            qp[4 * d + 2] = (hi & nc.mask_lo) | nc.magic_lo;
            qp[4 * d + 3] = (hi & nc.mask_hi) | nc.magic_hi;
        }
    }
}

__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {
    return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
}

// Eight consecutive scaled inputs -> the four packed pairs of one 16-byte LDS word.
template <int BITS>
__device__ __forceinline__ uint4 pack_inputs(const float* v) {
    if (BITS == 8) return make_uint4(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]), pack_h2(v[4], v[5]), pack_h2(v[6], v[7]));
    return make_uint4(pack_h2(v[0], v[4]), pack_h2(v[1], v[5]), pack_h2(v[2], v[6]), pack_h2(v[3], v[7]));
}

template <int ACT, bool XF32>
__device__ __forceinline__ void load8(const void* x, size_t off, float* v) {
    if (XF32) {
        const float4 a = *reinterpret_cast<const float4*>((const float*)x + off);
        const float4 b = *reinterpret_cast<const float4*>((const float*)x + off + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 a = *reinterpret_cast<const uint4*>((const uint16_t*)x + off);
        act2_to_f32<ACT>(a.x, v[0], v[1]); act2_to_f32<ACT>(a.y, v[2], v[3]);
        act2_to_f32<ACT>(a.z, v[4], v[5]); act2_to_f32<ACT>(a.w, v[6], v[7]);
    }
}

// Power of two that maps amax into [1024, 2048), and its inverse; 1 when amax is
// zero, denormal-small, infinite or NaN.
__device__ __forceinline__ void pow2_scale(float amax, float& sc, float& isc) {
    const uint32_t e = (__float_as_uint(amax) >> 23) & 0xFFu;
    if (e < 24u || e > 254u) { sc = 1.0f; isc = 1.0f; return; }
    sc = __uint_as_float((264u - e) << 23);      // 2^(10 - (e - 127))
    isc = __uint_as_float((e - 10u) << 23);      // 2^((e - 127) - 10)
}

// TOKS = 1: exactly one input, kept in registers for the whole block.  TOKS = 0:
// we.pair_count inputs (2..MAX_TOK), walked by a real loop inside each stage so
// that only one input's columns are live at a time.
// LDS: [ntok][n/8] uint4 packed inputs | [ntok][NCH*SEG][2] float chunk sums (all, odd pairs) |
//      [MAX_TOK*4] float wave maxima | [MAX_TOK] float inverse scales.
//
// MODE says where an entry's rows are named (entries made inside the launch that uses them read
// no pair tables).  ROWS_TABLES: p.pair_in / p.pair_out.  ROWS_DIRECT (one input only): input row
// we.reserved, output row we.pair_start.  ROWS_DENSE: input and output row we.pair_start + t, and
// the result goes to p.out (fp32) and / or p.out_act (16 bit), whichever is not null.
constexpr int ROWS_TABLES = 0, ROWS_DIRECT = 1, ROWS_DENSE = 2;
template <int ACT, int BITS, int SEG, int NCH, int TOKS, bool DUAL, bool XF32, int RPI, int ITERS, int MODE = ROWS_TABLES,
          bool PRENORM = false>
__device__ __forceinline__ void expert_rows_body(const RowsParams& p, const WorkEntry& we, uint32_t rb,
                                                 uint4* lds) {
    static_assert(!PRENORM || (MODE == ROWS_DENSE && !XF32), "the prologue is for dense launches over 16-bit rows");
    static_assert(MODE != ROWS_DIRECT || TOKS == 1, "a direct entry holds one input");
    auto in_row = [&](int t) -> uint32_t {
        return MODE == ROWS_DIRECT ? we.reserved : MODE == ROWS_DENSE ? we.pair_start + t : p.pair_in[we.pair_start + t];
    };
    auto out_row_of = [&](int t) -> uint32_t {
        return MODE == ROWS_DIRECT ? we.pair_start : MODE == ROWS_DENSE ? we.pair_start + t : p.pair_out[we.pair_start + t];
    };
    constexpr int EPC = Chunk<BITS>::elems;
    constexpr int PAIRS = EPC / 2;                // packed pairs per chunk
    constexpr int H = PAIRS / 4;                  // 16-byte LDS words per chunk
    constexpr int RPL = 64 / SEG;                 // rows per load instruction
    constexpr int ROWS_WAVE = RPL * RPI * ITERS;
    constexpr int WORDS_TOK = NCH * H * SEG;      // == n / 8
    static_assert(ITERS % 2 == 0, "ITERS must be even (double buffering)");
    using Stage = RowStage<BITS, SEG, NCH, DUAL, RPI>;
    const int ntok = TOKS ? TOKS : (int)we.pair_count;
    const NibbleConsts nib = nibble_consts();
    const uint8_t* blob = blob_ptr(p.src, we.expert);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int seg_id = lane / SEG, sl = lane % SEG;
    const uint32_t groups = p.n / NVMAI_GROUP;
    const uint32_t row_bytes = p.n * BITS / 8;
    const uint8_t* WA = blob + p.wA;
    const uint16_t* SA = reinterpret_cast<const uint16_t*>(blob + p.sA);
    const uint16_t* BA = reinterpret_cast<const uint16_t*>(blob + p.bA);
    const uint8_t* WB = DUAL ? blob + p.wB : nullptr;
    const uint16_t* SB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.sB) : nullptr;
    const uint16_t* BB = DUAL ? reinterpret_cast<const uint16_t*>(blob + p.bB) : nullptr;
    const uint32_t row_base = (rb * 4 + wave) * ROWS_WAVE;
    uint4* xw = lds;
    float* xs_tab = reinterpret_cast<float*>(lds + MAX_TOK * WORDS_TOK);
    float* wmax_tab = xs_tab + 2 * MAX_TOK * NCH * SEG;
    float* isc_tab = wmax_tab + MAX_TOK * 4;

    auto load_stage = [&](Stage& st, int it) {
#pragma unroll
        for (int i = 0; i < RPI; ++i) {
            const uint32_t row = row_base + (it * RPI + i) * RPL + seg_id;
            const uint32_t r = row < p.rows ? row : p.rows - 1;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                // a lane's chunks are neighbours (sl * NCH + c): with NCH * EPC <= 64 they share
                // one quantization group, whose scale and bias are then loaded once
                const uint32_t chunk = sl * NCH + c;
                const uint32_t g = chunk * EPC / NVMAI_GROUP;
                const bool fresh = c == 0 || NCH * EPC > NVMAI_GROUP;
                st.qa[i][c] = *reinterpret_cast<const uint4*>(WA + (size_t)r * row_bytes + chunk * 16);
                st.sa[i][c] = fresh ? SA[(size_t)r * groups + g] : st.sa[i][0];
                st.ba[i][c] = fresh ? BA[(size_t)r * groups + g] : st.ba[i][0];
                if (DUAL) {
                    st.qb[i][c] = *reinterpret_cast<const uint4*>(WB + (size_t)r * row_bytes + chunk * 16);
                    st.sb[i][c] = fresh ? SB[(size_t)r * groups + g] : st.sb[i][0];
                    st.bb[i][c] = fresh ? BB[(size_t)r * groups + g] : st.bb[i][0];
                }
            }
        }
    };

    Stage s0, s1;
    load_stage(s0, 0);                            // both in flight while the inputs are staged
    load_stage(s1, 1);

    if (p.n <= 256 * 8) {
        // ---- short rows: every thread holds its eight elements of every input, so the inputs
        // are read once, all loads in flight together, and scaled from registers
        constexpr int MT = TOKS ? TOKS : MAX_TOK;
        float v[MT][8], m[MT];
        const uint32_t e0 = threadIdx.x * 8;
        const bool live = e0 < p.n;
        if (PRENORM) {
            // the normed rows are made here, in LDS behind the engine's own arrays, and read from there
            uint16_t* xl = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(lds) + rows_fast_lds_base(p.n, NCH, SEG));
            uint16_t* raw = xl + (size_t)MAX_TOK * p.n;
            const PreNormArgs a{(const uint16_t*)p.x, p.x_stride, p.pre_delta, p.pre_delta_stride, p.pre_weight,
                                p.pre_hidden_out, p.pre_hidden_stride, p.pre_normed_out, p.pre_normed_stride, p.pre_eps, p.n};
            stage_prenorm_rows<ACT>(a, we.pair_start, (uint32_t)ntok, xl, raw, blockIdx.x == 0);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                if (t >= ntok) break;
                if (live) {
                    const uint4 r = *reinterpret_cast<const uint4*>(xl + (size_t)t * p.n + e0);
                    act2_to_f32<ACT>(r.x, v[t][0], v[t][1]); act2_to_f32<ACT>(r.y, v[t][2], v[t][3]);
                    act2_to_f32<ACT>(r.z, v[t][4], v[t][5]); act2_to_f32<ACT>(r.w, v[t][6], v[t][7]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            if (t >= ntok || PRENORM) break;
            if (live) load8<ACT, XF32>(p.x, (size_t)in_row(t) * p.x_stride + e0, v[t]);
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            if (t >= ntok) break;
            m[t] = 0.0f;
            if (live) {
#pragma unroll
                for (int j = 0; j < 8; ++j) m[t] = fmaxf(m[t], fabsf(v[t][j]));
            }
            m[t] = wave_max_f32(m[t]);
            if (lane == 0) wmax_tab[t * 4 + wave] = m[t];
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            if (t >= ntok) break;
            const float amax = fmaxf(fmaxf(wmax_tab[t * 4], wmax_tab[t * 4 + 1]),
                                     fmaxf(wmax_tab[t * 4 + 2], wmax_tab[t * 4 + 3]));
            float sc, isc;
            pow2_scale(amax, sc, isc);
            if (threadIdx.x == 0) isc_tab[t] = isc;
            if (live) {
#pragma unroll
                for (int j = 0; j < 8; ++j) v[t][j] *= sc;
                const uint32_t chunk = e0 / EPC, piece = (e0 % EPC) / 8;
                xw[t * WORDS_TOK + ((chunk % NCH) * H + piece) * SEG + (chunk / NCH)] = pack_inputs<BITS>(v[t]);
            }
        }
        __syncthreads();
    } else {
        // ---- pass 1: largest magnitude of every input row
    #pragma unroll 1
        for (int t = 0; t < ntok; ++t) {
            const size_t in_off = (size_t)in_row(t) * p.x_stride;
            float m = 0.0f;
            for (uint32_t e0 = threadIdx.x * 8; e0 < p.n; e0 += 256 * 8) {
                float v[8];
                load8<ACT, XF32>(p.x, in_off + e0, v);
    #pragma unroll
                for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(v[j]));
            }
            m = wave_max_f32(m);
            if (lane == 0) wmax_tab[t * 4 + wave] = m;
        }
        __syncthreads();
        // ---- pass 2: scale, convert, pack
    #pragma unroll 1
        for (int t = 0; t < ntok; ++t) {
            const size_t in_off = (size_t)in_row(t) * p.x_stride;
            const float amax = fmaxf(fmaxf(wmax_tab[t * 4], wmax_tab[t * 4 + 1]),
                                     fmaxf(wmax_tab[t * 4 + 2], wmax_tab[t * 4 + 3]));
            float sc, isc;
            pow2_scale(amax, sc, isc);
            if (threadIdx.x == 0) isc_tab[t] = isc;
            for (uint32_t e0 = threadIdx.x * 8; e0 < p.n; e0 += 256 * 8) {
                float v[8];
                load8<ACT, XF32>(p.x, in_off + e0, v);
    #pragma unroll
                for (int j = 0; j < 8; ++j) v[j] *= sc;
                const uint32_t chunk = e0 / EPC, piece = (e0 % EPC) / 8;
                xw[t * WORDS_TOK + ((chunk % NCH) * H + piece) * SEG + (chunk / NCH)] = pack_inputs<BITS>(v);
            }
        }
        __syncthreads();
    }
    // ---- chunk sums of the converted inputs, one thread per (input, chunk)
    for (int idx = threadIdx.x; idx < ntok * NCH * SEG; idx += 256) {
        const int t = idx / (NCH * SEG), cs = idx % (NCH * SEG), c = cs / SEG, l = cs % SEG;
        float sum = 0.0f, odd = 0.0f;                 // odd: the pairs 1, 3, 5, ... of the chunk
#pragma unroll
        for (int h = 0; h < H; ++h) {
            const uint4 w = xw[t * WORDS_TOK + (c * H + h) * SEG + l];
            const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const float both = f16_to_f32((uint16_t)(ws[d] & 0xFFFFu)) + f16_to_f32((uint16_t)(ws[d] >> 16));
                sum += both;
                if (d & 1) odd += both;
            }
        }
        xs_tab[(t * NCH * SEG + c * SEG + l) * 2] = sum;
        xs_tab[(t * NCH * SEG + c * SEG + l) * 2 + 1] = odd;
    }
    __syncthreads();

    auto compute_stage = [&](const Stage& st, int it) {
        uint32_t qpa[RPI][NCH][PAIRS], qpb[DUAL ? RPI : 1][NCH][PAIRS];
#pragma unroll
        for (int i = 0; i < RPI; ++i)
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                unpack_pairs<BITS>(st.qa[i][c], qpa[i][c], nib);
                if (DUAL) unpack_pairs<BITS>(st.qb[i][c], qpb[i][c], nib);
            }
#pragma unroll 1
        for (int t = 0; t < ntok; ++t) {
            uint32_t xp[NCH][PAIRS];
            float xs[NCH], xo[NCH];
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
#pragma unroll
                for (int h = 0; h < H; ++h) {
                    const uint4 w = xw[t * WORDS_TOK + (c * H + h) * SEG + sl];
                    xp[c][4 * h] = w.x; xp[c][4 * h + 1] = w.y; xp[c][4 * h + 2] = w.z; xp[c][4 * h + 3] = w.w;
                }
                const float2 two = *reinterpret_cast<const float2*>(&xs_tab[(t * NCH * SEG + c * SEG + sl) * 2]);
                xs[c] = two.x;
                xo[c] = two.y;
            }
            const float isc = isc_tab[t];
            const uint32_t out_row = out_row_of(t);
#pragma unroll
            for (int i = 0; i < RPI; ++i) {
                const uint32_t row = row_base + (it * RPI + i) * RPL + seg_id;
                float accA = 0.0f, accB = 0.0f;
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    float dotA = 0.0f, dotB = 0.0f;
#pragma unroll
                    for (int m = 0; m < PAIRS; ++m) {
                        dotA = dot2_acc(qpa[i][c][m], xp[c][m], dotA);
                        if (DUAL) dotB = dot2_acc(qpb[i][c][m], xp[c][m], dotB);
                    }
                    dotA = fmaf(-1024.0f, xs[c], dotA);
                    if (BITS == 4) dotA = fmaf(ODD_PAIR_OFFSET_GAP, xo[c], dotA);
                    accA = fmaf(bf16_to_f32(st.sa[i][c]), dotA, accA);
                    accA = fmaf(bf16_to_f32(st.ba[i][c]), xs[c], accA);
                    if (DUAL) {
                        dotB = fmaf(-1024.0f, xs[c], dotB);
                        if (BITS == 4) dotB = fmaf(ODD_PAIR_OFFSET_GAP, xo[c], dotB);
                        accB = fmaf(bf16_to_f32(st.sb[i][c]), dotB, accB);
                        accB = fmaf(bf16_to_f32(st.bb[i][c]), xs[c], accB);
                    }
                }
                const float a = seg_reduce_sum<SEG>(accA) * isc;
                float v = a;
                if (DUAL) {
                    const float u = seg_reduce_sum<SEG>(accB) * isc;
                    v = silu_fast(a) * u; // moe.metal:134-139 (silu branch), CPUExpertFFN.swift:122-124
                }
                if (seg_result_lane<SEG>(lane) && row < p.rows) {
                    if (MODE != ROWS_DENSE || p.out) p.out[(size_t)out_row * p.out_stride + row] = v;
                    if (MODE == ROWS_DENSE && p.out_act)
                        ((uint16_t*)p.out_act)[(size_t)out_row * p.out_act_stride + row] = f32_to_act<ACT>(v);
                }
            }
        }
    };

    // Unrolled on purpose: as a real loop its two conditional loads meet at the back edge, the
    // compiler can no longer tell how many loads are in flight behind the stage about to be
    // used, and waits for all of them -- the stage just requested included.
#pragma unroll
    for (int it = 0; it < ITERS; it += 2) {
        compute_stage(s0, it);
        if (it + 2 < ITERS) load_stage(s0, it + 2);
        compute_stage(s1, it + 1);
        if (it + 3 < ITERS) load_stage(s1, it + 3);
    }
}

// Bytes of dynamic LDS the fast engine needs for rows of n codes; with the prologue the normed rows
// (MAX_TOK x n) and one raw row follow at a 16-byte boundary.
__host__ __device__ inline size_t rows_fast_lds_bytes(uint32_t n, int nch, int seg) {
    return (size_t)MAX_TOK * (n / 8) * 16 + (size_t)MAX_TOK * nch * seg * 8 + MAX_TOK * 4 * 4 + MAX_TOK * 4;
}
__host__ __device__ inline size_t rows_fast_lds_bytes_prenorm(uint32_t n, int nch, int seg) {
    return rows_fast_lds_base(n, nch, seg) + (size_t)(MAX_TOK + 1) * n * 2;
}

// MAXTOK = 1: single-input launches.  MAXTOK = 4: the body is chosen by the
// entry's pair count (uniform per block), so an expert routed to by one token
// does not pay for more.
// DENSE: the matrix in blob slot 0 against the input rows 0 .. dense_count - 1, entry e = the
// rows e * MAXTOK .. (a grid of exactly that many entries; no work list, no pair tables).
template <int ACT, int BITS, int SEG, int NCH, int MAXTOK, bool DUAL, bool XF32, int RPI, int ITERS, bool DENSE = false,
          bool PRENORM = false>
__global__ __launch_bounds__(256) void expert_rows_fast(RowsParams p) {
    extern __shared__ uint4 rows_lds[];
    const uint32_t entry = blockIdx.x / p.blocks_per_entry;
    const uint32_t rb = blockIdx.x % p.blocks_per_entry;
    constexpr int MODE = DENSE ? ROWS_DENSE : ROWS_TABLES;
    WorkEntry we;
    if (DENSE) {
        we.expert = NVMAI_SLOT_FLAG;
        we.pair_start = entry * MAXTOK;
        we.pair_count = min((uint32_t)MAXTOK, p.dense_count - entry * MAXTOK);
        we.reserved = 0;
    } else {
        if (entry >= *p.n_entries) return;
        we = p.entries[entry];
    }
    if (MAXTOK == 1 || we.pair_count == 1)
        expert_rows_body<ACT, BITS, SEG, NCH, 1, DUAL, XF32, RPI, ITERS, MODE, PRENORM>(p, we, rb, rows_lds);
    else
        expert_rows_body<ACT, BITS, SEG, NCH, 0, DUAL, XF32, RPI, ITERS, MODE, PRENORM>(p, we, rb, rows_lds);
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
    int x_vec;                     // rows of x (and eff_scale) are 16-byte aligned
    const uint16_t* eff_scale;     // optional bf16 [d]
    uint32_t x_stride, tokens, num_experts, d;
    float* logits;                 // [tokens, num_experts]
    float* gate_logit;             // [tokens]
    // Optional prologue (pre_weight != null): x holds the residual stream's rows and the block's
    // input row is rmsnorm(round(x + pre_delta)) * pre_weight, computed by every block for itself
    // with the arithmetic of residual_add_rmsnorm_kernel (same bits); the block of the first rows
    // also stores the updated residual row to pre_hidden_out (not x: other blocks still read it)
    // and the normed row to pre_normed_out for the kernels that follow.  Rows 16-byte aligned.
    const uint16_t* pre_delta;     // [tokens, pre_delta_stride], may be null (norm only)
    const uint16_t* pre_weight;    // BF16 [d]
    uint16_t* pre_hidden_out;      // [tokens, pre_hidden_stride]
    uint16_t* pre_normed_out;      // [tokens, pre_normed_stride]
    uint32_t pre_delta_stride, pre_hidden_stride, pre_normed_stride;
    float pre_eps;
};

// Tokens per block in y.  One: the launch is a chain of latencies (stage the row, load eight
// weight rows, sum, butterfly), so more blocks with less to do each finish sooner than fewer
// blocks walking several tokens (measured at 32 tokens: 11.7 us with four, 9.0 with two or one;
// at four tokens 10.4 -> 6.6 us).  The weight rows are re-read per token from L2.
constexpr int ROUTER_TOK = 1;

// EPC consecutive activations of one row as floats, optionally times the bf16
// effective scale (one rounding, as moe.metal:200-201 multiplies before use).
template <int ACT, int EPC>
__device__ __forceinline__ void router_x_from_raw(const RouterParams& p, const uint4* raw, uint32_t e0, float* xv) {
#pragma unroll
    for (int i = 0; i < EPC / 8; ++i) {
        act2_to_f32<ACT>(raw[i].x, xv[8 * i], xv[8 * i + 1]);
        act2_to_f32<ACT>(raw[i].y, xv[8 * i + 2], xv[8 * i + 3]);
        act2_to_f32<ACT>(raw[i].z, xv[8 * i + 4], xv[8 * i + 5]);
        act2_to_f32<ACT>(raw[i].w, xv[8 * i + 6], xv[8 * i + 7]);
    }
    if (p.eff_scale) {
#pragma unroll
        for (int j = 0; j < EPC; ++j) xv[j] = __fmul_rn(xv[j], bf16_to_f32(p.eff_scale[e0 + j]));
    }
}

// The block's token rows, as stored, into LDS ([nt][d] 16-bit): the eight rows of a block read
// the same inputs, and reading them from LDS when they are used keeps only the weights in
// registers.  Ends with a barrier.
__device__ __forceinline__ void router_stage_x(const RouterParams& p, uint32_t t0, uint32_t nt, uint16_t* xl) {
    if (p.x_vec) {
        const uint32_t per_row = p.d / 8;
        for (uint32_t i = threadIdx.x; i < nt * per_row; i += 256) {
            const uint32_t t = i / per_row, c = i % per_row;
            reinterpret_cast<uint4*>(xl)[i] =
                *reinterpret_cast<const uint4*>((const uint16_t*)p.x + (size_t)(t0 + t) * p.x_stride + c * 8);
        }
    } else {                       // unaligned rows (e.g. a padded hidden stride): element loads
        for (uint32_t i = threadIdx.x; i < nt * p.d; i += 256)
            xl[i] = ((const uint16_t*)p.x)[(size_t)(t0 + i / p.d) * p.x_stride + i % p.d];
    }
    __syncthreads();
}

// The same with the prologue (stage_prenorm_rows): the block's rows are summed with their delta,
// normed and staged.
template <int ACT>
__device__ __forceinline__ void router_stage_prenorm(const RouterParams& p, uint32_t t0, uint32_t nt, uint16_t* xl,
                                                     uint16_t* raw) {
    const PreNormArgs a{(const uint16_t*)p.x, p.x_stride, p.pre_delta, p.pre_delta_stride, p.pre_weight, p.pre_hidden_out,
                        p.pre_hidden_stride, p.pre_normed_out, p.pre_normed_stride, p.pre_eps, p.d};
    stage_prenorm_rows<ACT>(a, t0, nt, xl, raw, blockIdx.x == 0);
}

// One row against up to ROUTER_TOK tokens; hl = lane in the half-wave, CPL =
// chunks per lane (compile time) so that every load is issued before the first
// use: a dependent round trip to HBM costs more than the whole arithmetic.
// Per token the lane accumulates over its chunks in ascending order.
// A half-wave's share of one weight row, fetched before the inputs are staged: the two do not depend
// on each other, and a trip to memory costs more than the arithmetic that follows.
template <int CPL>
struct RouterRowRegs { uint4 w[CPL]; uint16_t s[CPL], b[CPL]; };

template <int CPL>
__device__ __forceinline__ void router_row_prefetch(const RouterParams& p, const RowsDesc& r, uint32_t row, int hl,
                                                    RouterRowRegs<CPL>& g) {
    const uint32_t epc = r.kind == 16 ? 8u : (r.kind == 8 ? 16u : 32u);
    const uint32_t chunks = p.d / epc, groups = p.d / NVMAI_GROUP;
    const uint8_t* wr = (const uint8_t*)r.w + (size_t)row * ((size_t)p.d * r.kind / 8);
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        const uint32_t c = hl + 32 * i;
        if (c < chunks) {
            g.w[i] = *reinterpret_cast<const uint4*>(wr + (size_t)c * 16);
            if (r.kind != 16) {
                const uint32_t gi = c * epc / NVMAI_GROUP;
                g.s[i] = r.s[(size_t)row * groups + gi];
                g.b[i] = r.b[(size_t)row * groups + gi];
            }
        }
    }
}

template <int ACT, int KIND, int CPL>
__device__ __forceinline__ void router_row_dots(const RouterParams& p, const RouterRowRegs<CPL>& g,
                                                const uint16_t* xl, uint32_t nt, int hl, float* acc) {
    constexpr int EPC = KIND == 16 ? 8 : (KIND == 8 ? 16 : 32);
    constexpr int XV = EPC / 8;
    const uint32_t chunks = p.d / EPC;
#pragma unroll
    for (int t = 0; t < ROUTER_TOK; ++t) acc[t] = 0.0f;
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        const uint32_t c = hl + 32 * i;
        if (c >= chunks) break;
        float q[EPC];
        if (KIND == 16) {
            act2_to_f32<ACT_BF16>(g.w[i].x, q[0], q[1]); act2_to_f32<ACT_BF16>(g.w[i].y, q[2], q[3]);
            act2_to_f32<ACT_BF16>(g.w[i].z, q[4], q[5]); act2_to_f32<ACT_BF16>(g.w[i].w, q[6], q[7]);
        } else {
            unpack_chunk<KIND == 16 ? 8 : KIND>(g.w[i], q);
        }
#pragma unroll
        for (int t = 0; t < ROUTER_TOK; ++t) {
            if ((uint32_t)t >= nt) break;
            float xv[EPC];
            uint4 xraw[XV];
#pragma unroll
            for (int v = 0; v < XV; ++v) xraw[v] = *reinterpret_cast<const uint4*>(xl + (size_t)t * p.d + c * EPC + 8 * v);
            router_x_from_raw<ACT, EPC>(p, xraw, c * EPC, xv);
            if (KIND == 16) {
#pragma unroll
                for (int j = 0; j < EPC; ++j) acc[t] = fmaf(q[j], xv[j], acc[t]);
            } else {
                float dot = 0.0f, xs = 0.0f;
#pragma unroll
                for (int j = 0; j < EPC; ++j) {
                    dot = fmaf(q[j], xv[j], dot);
                    xs = __fadd_rn(xs, xv[j]);
                }
                acc[t] = fmaf(bf16_to_f32(g.s[i]), dot, acc[t]);
                acc[t] = fmaf(bf16_to_f32(g.b[i]), xs, acc[t]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < ROUTER_TOK; ++t)
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) acc[t] = __fadd_rn(acc[t], shfl_xor_f(acc[t], off));
}

template <int ACT, int CPL>
__device__ __forceinline__ void router_row_any(const RouterParams& p, int kind, const RouterRowRegs<CPL>& g,
                                               const uint16_t* xl, uint32_t nt, int hl, float* acc) {
    if (kind == 16) router_row_dots<ACT, 16, CPL>(p, g, xl, nt, hl, acc);
    else if (kind == 8) router_row_dots<ACT, 8, CPL>(p, g, xl, nt, hl, acc);
    else router_row_dots<ACT, 4, CPL>(p, g, xl, nt, hl, acc);
}

// Largest chunk count per lane over the router and gate rows must be <= CPL.
template <int ACT, int CPL>
__global__ __launch_bounds__(256) void router_logits_kernel(RouterParams p) {
    extern __shared__ uint4 router_lds[];
    const uint16_t* xl = reinterpret_cast<const uint16_t*>(router_lds);
    const int hw = threadIdx.x >> 5, hl = threadIdx.x & 31;
    const uint32_t row = blockIdx.x * 8 + hw;
    const uint32_t total_rows = p.num_experts + (p.gate.kind ? 1u : 0u);
    const uint32_t t0 = blockIdx.y * ROUTER_TOK;
    const uint32_t nt = min((uint32_t)ROUTER_TOK, p.tokens - t0);
    const bool live = row < total_rows, is_gate = row >= p.num_experts;
    const RowsDesc& rd = is_gate ? p.gate : p.router;
    RouterRowRegs<CPL> g;
    if (live) router_row_prefetch<CPL>(p, rd, is_gate ? 0u : row, hl, g);      // in flight while the inputs are staged
    if (p.pre_weight) {
        uint16_t* raw = reinterpret_cast<uint16_t*>(router_lds) + (size_t)ROUTER_TOK * p.d;
        router_stage_prenorm<ACT>(p, t0, nt, reinterpret_cast<uint16_t*>(router_lds), raw);
    } else {
        router_stage_x(p, t0, nt, reinterpret_cast<uint16_t*>(router_lds));
    }
    if (!live) return;                               // uniform per half-wave
    float acc[ROUTER_TOK];
    router_row_any<ACT, CPL>(p, rd.kind, g, xl, nt, hl, acc);
    if (hl == 0) {
        for (uint32_t t = 0; t < nt; ++t) {
            if (is_gate) p.gate_logit[t0 + t] = acc[t];
            else p.logits[(size_t)(t0 + t) * p.num_experts + row] = acc[t];
        }
    }
}

// ---- router logits for many tokens ---------------------------------------------------------
// The same sums in the same order as router_logits_kernel, so the logits are the same bits and
// the routing does not depend on which kernel ran; only the tiling differs.  A half-wave owns R
// rows against the block's RT_TOK tokens: a chunk of each row is converted to floats once and
// then used by every token, and a token's chunk once for the R rows, instead of once per
// (row, token) pair.  The inputs of the block sit in LDS as stored.  One launch per matrix (the
// router rows, then the single gate row) because their formats may differ.
constexpr int RT_TOK = 8;

// EFF: the inputs are multiplied by the bf16 effective scale (a compile-time switch: a branch per
// token in the loop body makes the compiler convert all sixteen tokens' chunks before the first
// multiply-add, and the accumulators no longer fit beside them).
template <int ACT, int KIND, bool EFF>
__global__ __launch_bounds__(256, KIND == 16 ? 4 : 2) void router_logits_tiled_kernel(RouterParams p, RowsDesc r, uint32_t n_rows,
                                                                  float* out, uint32_t out_ld) {
    constexpr int EPC = KIND == 16 ? 8 : (KIND == 8 ? 16 : 32);
    constexpr int XV = EPC / 8;
    constexpr int R = KIND == 4 ? 2 : 4;             // rows per half-wave: what the register file holds at four blocks per CU
                                                     // (eight BF16 rows, 174 registers, two blocks: 117 against 91 us at 4096 tokens)
    extern __shared__ uint4 router_lds[];
    const uint16_t* xl = reinterpret_cast<const uint16_t*>(router_lds);
    const int hw = threadIdx.x >> 5, hl = threadIdx.x & 31;
    const uint32_t row0 = (blockIdx.x * 8 + hw) * R;
    const uint32_t t0 = blockIdx.y * RT_TOK;
    const uint32_t nt = min((uint32_t)RT_TOK, p.tokens - t0);
    const uint32_t chunks = p.d / EPC;
    const uint32_t groups = p.d / NVMAI_GROUP;
    const size_t row_bytes = (size_t)p.d * KIND / 8;
    // the rows' chunks one iteration ahead of their use (the first ones while the inputs are staged):
    // rows past the end repeat the last one, chunks past the end the lane's last one, both unused
    uint4 wnext[R];
    uint16_t snext[R], bnext[R];
    auto fetch_rows = [&](uint32_t c) {
        const uint32_t cc = min(c, chunks - 1u);
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint32_t row = min(row0 + i, n_rows - 1);
            wnext[i] = *reinterpret_cast<const uint4*>((const uint8_t*)r.w + row * row_bytes + (size_t)cc * 16);
            if (KIND != 16) {
                const uint32_t g = cc * EPC / NVMAI_GROUP;
                snext[i] = r.s[(size_t)row * groups + g];
                bnext[i] = r.b[(size_t)row * groups + g];
            }
        }
    };
    fetch_rows(hl);
    router_stage_x(p, t0, nt, reinterpret_cast<uint16_t*>(router_lds));
    if (row0 >= n_rows) return;                      // uniform per half-wave
    float acc[R][RT_TOK];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int t = 0; t < RT_TOK; ++t) acc[i][t] = 0.0f;
#pragma unroll 1
    for (uint32_t c = hl; c < chunks; c += 32) {
        float q[R][EPC], sc[R], bi[R];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint4 w = wnext[i];
            if (KIND == 16) {
                act2_to_f32<ACT_BF16>(w.x, q[i][0], q[i][1]); act2_to_f32<ACT_BF16>(w.y, q[i][2], q[i][3]);
                act2_to_f32<ACT_BF16>(w.z, q[i][4], q[i][5]); act2_to_f32<ACT_BF16>(w.w, q[i][6], q[i][7]);
            } else {
                unpack_chunk<KIND == 16 ? 8 : KIND>(w, q[i]);
                sc[i] = bf16_to_f32(snext[i]);
                bi[i] = bf16_to_f32(bnext[i]);
            }
        }
        fetch_rows(c + 32);
        float eff[EFF ? EPC : 1];
        if (EFF) {
#pragma unroll
            for (int j = 0; j < EPC; ++j) eff[j] = bf16_to_f32(p.eff_scale[c * EPC + j]);
        }
        // rows of LDS past the block's last token hold whatever they held: their sums are never stored
        uint4 xnext[XV];
#pragma unroll
        for (int v = 0; v < XV; ++v) xnext[v] = *reinterpret_cast<const uint4*>(xl + c * EPC + 8 * v);
#pragma unroll
        for (int t = 0; t < RT_TOK; ++t) {
            float xv[EPC];
            uint4 xraw[XV];
#pragma unroll
            for (int v = 0; v < XV; ++v) xraw[v] = xnext[v];
            if (t + 1 < RT_TOK) {                        // the next token's chunk is under way during this one's sums
#pragma unroll
                for (int v = 0; v < XV; ++v)
                    xnext[v] = *reinterpret_cast<const uint4*>(xl + (size_t)(t + 1) * p.d + c * EPC + 8 * v);
            }
#pragma unroll
            for (int v = 0; v < XV; ++v) {
                act2_to_f32<ACT>(xraw[v].x, xv[8 * v], xv[8 * v + 1]);
                act2_to_f32<ACT>(xraw[v].y, xv[8 * v + 2], xv[8 * v + 3]);
                act2_to_f32<ACT>(xraw[v].z, xv[8 * v + 4], xv[8 * v + 5]);
                act2_to_f32<ACT>(xraw[v].w, xv[8 * v + 6], xv[8 * v + 7]);
            }
            if (EFF) {                                   // one rounding, as moe.metal:200-201 multiplies before use
#pragma unroll
                for (int j = 0; j < EPC; ++j) xv[j] = __fmul_rn(xv[j], eff[j]);
            }
            if (KIND == 16) {
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int j = 0; j < EPC; ++j) acc[i][t] = fmaf(q[i][j], xv[j], acc[i][t]);
            } else {
                float xs = 0.0f;
#pragma unroll
                for (int j = 0; j < EPC; ++j) xs = __fadd_rn(xs, xv[j]);
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    float dot = 0.0f;
#pragma unroll
                    for (int j = 0; j < EPC; ++j) dot = fmaf(q[i][j], xv[j], dot);
                    acc[i][t] = fmaf(sc[i], dot, acc[i][t]);
                    acc[i][t] = fmaf(bi[i], xs, acc[i][t]);
                }
            }
            // one token at a time: without the fence the scheduler fetches every token's chunk up
            // front and the accumulators no longer fit beside them
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int t = 0; t < RT_TOK; ++t) {
#pragma unroll
            for (int off = 16; off >= 1; off >>= 1) acc[i][t] = __fadd_rn(acc[i][t], shfl_xor_f(acc[i][t], off));
            if (hl == 0 && (uint32_t)t < nt && row0 + i < n_rows) out[(size_t)(t0 + t) * out_ld + row0 + i] = acc[i][t];
            if ((t & 3) == 3) __builtin_amdgcn_sched_barrier(0);     // four butterflies in flight, not all 64
        }
}

// One row (the shared expert's gate row) against many tokens: a half-wave per token, its inputs read
// straight from memory (16 bytes per lane and load; nothing is shared between tokens but the one row,
// which every half-wave reads from cache), all of a lane's loads requested before the first sum.  The
// same sums in the same order as the kernels above, so the same bits.  Rows of x 16-byte aligned.
template <int ACT, int KIND, int CPL>
__global__ __launch_bounds__(256) void router_single_row_kernel(RouterParams p, RowsDesc r, float* out, uint32_t out_ld) {
    constexpr int EPC = KIND == 16 ? 8 : (KIND == 8 ? 16 : 32);
    constexpr int XV = EPC / 8;
    const int hw = threadIdx.x >> 5, hl = threadIdx.x & 31;
    const uint32_t t = blockIdx.x * 8 + hw;
    if (t >= p.tokens) return;                       // uniform per half-wave
    const uint32_t chunks = p.d / EPC;
    const uint16_t* xrow = (const uint16_t*)p.x + (size_t)t * p.x_stride;
    uint4 wv[CPL], xraw[CPL][XV];
    uint16_t sv[CPL], bv[CPL];
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        const uint32_t c = min((uint32_t)hl + 32u * i, chunks - 1u);      // past the end: the last chunk again, unused
        wv[i] = *reinterpret_cast<const uint4*>((const uint8_t*)r.w + (size_t)c * 16);
#pragma unroll
        for (int v = 0; v < XV; ++v) xraw[i][v] = *reinterpret_cast<const uint4*>(xrow + c * EPC + 8 * v);
        if (KIND != 16) {
            sv[i] = r.s[c * EPC / NVMAI_GROUP];
            bv[i] = r.b[c * EPC / NVMAI_GROUP];
        }
    }
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        const uint32_t c = hl + 32u * i;
        if (c < chunks) {
            float q[EPC], xv[EPC];
            if (KIND == 16) {
                act2_to_f32<ACT_BF16>(wv[i].x, q[0], q[1]); act2_to_f32<ACT_BF16>(wv[i].y, q[2], q[3]);
                act2_to_f32<ACT_BF16>(wv[i].z, q[4], q[5]); act2_to_f32<ACT_BF16>(wv[i].w, q[6], q[7]);
            } else {
                unpack_chunk<KIND == 16 ? 8 : KIND>(wv[i], q);
            }
            router_x_from_raw<ACT, EPC>(p, xraw[i], c * EPC, xv);
            if (KIND == 16) {
#pragma unroll
                for (int j = 0; j < EPC; ++j) acc = fmaf(q[j], xv[j], acc);
            } else {
                float dot = 0.0f, xs = 0.0f;
#pragma unroll
                for (int j = 0; j < EPC; ++j) {
                    dot = fmaf(q[j], xv[j], dot);
                    xs = __fadd_rn(xs, xv[j]);
                }
                acc = fmaf(bf16_to_f32(sv[i]), dot, acc);
                acc = fmaf(bf16_to_f32(bv[i]), xs, acc);
            }
        }
    }
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) acc = __fadd_rn(acc, shfl_xor_f(acc, off));
    if (hl == 0) out[(size_t)t * out_ld] = acc;
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

// Selection for token t by one wave: lane r < top_k ends with the r-th best (score, index).
__device__ __forceinline__ void select_topk_core(const SelectParams& p, uint32_t t, int lane, float& my_score,
                                                 uint32_t& my_idx) {
    float val[TOPK_MAX_PER_LANE];
    bool taken[TOPK_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < TOPK_MAX_PER_LANE; ++j) {
        const uint32_t e = lane + 64 * j;
        const size_t at = (size_t)t * p.num_experts + e;
        val[j] = e >= p.num_experts ? 0.0f : p.logits[at];
        taken[j] = e >= p.num_experts;
    }
    my_score = 0.0f;
    my_idx = 0;
    for (uint32_t round = 0; round < p.top_k; ++round) {
        float bv = -INFINITY;
        uint32_t bi = 0xFFFFFFFFu;
#pragma unroll
        for (int j = 0; j < TOPK_MAX_PER_LANE; ++j) {
            const uint32_t e = lane + 64 * j;
            if (!taken[j] && (bi == 0xFFFFFFFFu || better(val[j], e, bv, bi))) { bv = val[j]; bi = e; }
        }
        // wave argmax: highest value, lowest index among equals
        const float wm = wave_max_f32(bi == 0xFFFFFFFFu ? -INFINITY : bv);
        bi = wave_min_u32((bi != 0xFFFFFFFFu && bv == wm) ? bi : 0xFFFFFFFFu);
        bv = wm;
        if (bi == 0xFFFFFFFFu) { bi = 0; bv = -INFINITY; }   // fewer candidates than k
#pragma unroll
        for (int j = 0; j < TOPK_MAX_PER_LANE; ++j)
            if ((uint32_t)(lane + 64 * j) == bi) taken[j] = true;
        if ((uint32_t)lane == round) { my_score = bv; my_idx = bi; }
    }
}

// Softmax over the selected scores (in the lanes below top_k) times the expert's gain; stores
// index and fp16 weight of token t.
__device__ __forceinline__ void select_store_routes(const SelectParams& p, uint32_t t, int lane, float my_score,
                                                    uint32_t my_idx) {
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

__device__ void select_topk_wave(const SelectParams& p, uint32_t t, int lane) {
    float my_score;
    uint32_t my_idx;
    select_topk_core(p, t, lane, my_score, my_idx);
    select_store_routes(p, t, lane, my_score, my_idx);
}

__global__ __launch_bounds__(256) void select_topk_kernel(SelectParams p) {
    const uint32_t t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t < p.tokens) select_topk_wave(p, t, threadIdx.x & 63);
}

// ---- decode work list --------------------------------------------------------------
// Top-k for every token of a small decode batch (one wave per token, four per
// block), then the block that finishes last groups the (token, slot) pairs by
// expert so that each distinct expert is streamed once, and appends the shared
// expert over all tokens.  Entries are ordered heaviest first (shared expert, then
// routed entries by pair count 4, 3, 2, 1) so that the long blocks start early.
// The order of pairs and entries inside a class comes from LDS atomics and may
// differ between runs; every pair's arithmetic is independent of it, so the
// results do not.
struct GroupParams {
    SelectParams sel;
    uint32_t tok_per_entry;    // 1..MAX_TOK
    int has_shared;
    WorkEntry* entries;
    uint32_t* n_entries;       // [0] = entries, [1] = distinct experts
    uint32_t* stats;           // optional copy of n_entries[0..1]
    uint32_t* pair_token;      // input row per pair for phase 1
    uint32_t* pair_id;         // act / partial row per pair
    uint32_t* ticket;          // zero between launches; counts finished blocks
};

// The work list from every token's routed experts; one block, after all indices are written.
__device__ void build_work_list(const GroupParams& p, uint32_t* lds) {
    const uint32_t tokens = p.sel.tokens, top_k = p.sel.top_k, E = p.sel.num_experts;
    const uint32_t n_pairs = tokens * top_k;
    const uint32_t tid = threadIdx.x;
    uint32_t* cnt = lds;                  // [E] pairs per expert
    uint32_t* start = lds + E;            // [E] first pair of the expert
    uint32_t* slotf = lds + 2 * E;        // [E] first full entry of the expert inside its class
    uint32_t* slotr = lds + 3 * E;        // [E] remainder entry of the expert inside its class
    uint32_t* misc = lds + 4 * E;         // [0] pair cursor, [1..4] entries per class, [5] distinct
    uint32_t* rank = lds + 4 * E + 8;     // [n_pairs] rank of the pair inside its expert
    const volatile uint32_t* idx = p.sel.out_idx;   // written by other blocks: read past L1
    for (uint32_t i = tid; i < 4 * E + 8; i += blockDim.x) lds[i] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < n_pairs; i += blockDim.x) rank[i] = atomicAdd(&cnt[idx[i]], 1u);
    __syncthreads();
    const uint32_t tpe = p.tok_per_entry;
    for (uint32_t e = tid; e < E; e += blockDim.x) {
        const uint32_t c = cnt[e];
        if (!c) continue;
        start[e] = atomicAdd(&misc[0], c);
        atomicAdd(&misc[5], 1u);
        const uint32_t full = c / tpe, rem = c % tpe;
        if (full) slotf[e] = atomicAdd(&misc[tpe], full);
        if (rem) slotr[e] = atomicAdd(&misc[rem], 1u);
    }
    __syncthreads();
    const uint32_t shared_ent = p.has_shared ? (tokens + tpe - 1) / tpe : 0;
    uint32_t base[MAX_TOK + 1];
    uint32_t run = shared_ent;
    for (int c = MAX_TOK; c >= 1; --c) { base[c] = run; run += misc[c]; }
    const uint32_t total_ent = run;
    for (uint32_t e = tid; e < E; e += blockDim.x) {
        const uint32_t c = cnt[e];
        if (!c) continue;
        const uint32_t full = c / tpe, rem = c % tpe;
        for (uint32_t j = 0; j < full; ++j)
            p.entries[base[tpe] + slotf[e] + j] = WorkEntry{e, start[e] + j * tpe, tpe, 0};
        if (rem) p.entries[base[rem] + slotr[e]] = WorkEntry{e, start[e] + full * tpe, rem, 0};
    }
    for (uint32_t i = tid; i < n_pairs; i += blockDim.x) {
        const uint32_t pos = start[idx[i]] + rank[i];
        p.pair_token[pos] = i / top_k;
        p.pair_id[pos] = i;
    }
    if (p.has_shared) {
        for (uint32_t j = tid; j < shared_ent; j += blockDim.x)
            p.entries[j] = WorkEntry{NVMAI_SLOT_FLAG | 8u, n_pairs + j * tpe, min(tpe, tokens - j * tpe), 0};
        for (uint32_t t = tid; t < tokens; t += blockDim.x) {
            p.pair_token[n_pairs + t] = t;
            p.pair_id[n_pairs + t] = n_pairs + t;
        }
    }
    if (tid == 0) {
        p.n_entries[0] = total_ent;
        p.n_entries[1] = misc[5];
        if (p.stats) { p.stats[0] = total_ent; p.stats[1] = misc[5]; }
        *p.ticket = 0;                    // ready for the next launch
    }
}

__global__ __launch_bounds__(256) void select_group_kernel(GroupParams p) {
    extern __shared__ uint32_t lds[];
    const uint32_t tokens = p.sel.tokens;
    const uint32_t tid = threadIdx.x;
    {
        const uint32_t t = blockIdx.x * 4 + (tid >> 6);
        if (t < tokens) select_topk_wave(p.sel, t, tid & 63);
    }
    __threadfence();                      // this block's indices are visible device-wide
    __syncthreads();
    if (tid == 0) lds[0] = atomicAdd(p.ticket, 1u);
    __syncthreads();
    if (lds[0] != gridDim.x - 1) return;  // uniform per block
    __syncthreads();
    build_work_list(p, lds);
}

// The same for at most four tokens in ONE block: nothing crosses a block, so the device-scope
// release of the multi-block kernel (an L2 write-back on this multi-die part) and its ticket
// are not needed.
__global__ __launch_bounds__(256) void select_group_one_block_kernel(GroupParams p) {
    extern __shared__ uint32_t lds[];
    const uint32_t t = threadIdx.x >> 6;
    if (t < p.sel.tokens) select_topk_wave(p.sel, t, threadIdx.x & 63);
    __syncthreads();
    build_work_list(p, lds);
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

// The combine, the residual add that follows the MoE block and the RMSNorm that opens the next block, one
// block per token: acc as combine_kernel takes it (same terms, same order), y = round(acc) (stored when
// asked for), hidden = round(hidden + y) in place, normed = rmsnorm(hidden) * weight with the stated
// summation order of rms_wave_sum / rms_inverse -- the bits of combine_kernel followed by the
// residual-add-norm kernel.  d a multiple of 8, at most 8192; rows 16-byte aligned.
struct PostNormArgs {
    uint16_t* hidden; uint32_t hidden_stride;      // residual stream, updated in place
    const uint16_t* weight; float eps;             // BF16 [d]
    uint16_t* normed; uint32_t normed_stride;
};

template <int ACT>
__global__ __launch_bounds__(256) void combine_postnorm_kernel(CombineParams p, PostNormArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint16_t post_raw[];
    const uint32_t t = blockIdx.x, per_row = p.d / 8, lane = threadIdx.x & 63;
    uint4 v[ROUTER_PRE_PIECES], wv[ROUTER_PRE_PIECES];
    // the gate logit is requested like every other input, unconditionally (a load under a condition is
    // waited for on the spot, ahead of everything after it); without a gate the word read is not used
    const float gate_in = *(p.has_shared && p.gate_logit ? p.gate_logit + t : p.partials);
#pragma unroll
    for (int k = 0; k < ROUTER_PRE_PIECES; ++k) {
        const uint32_t c = threadIdx.x + 256 * k;
        if (c >= per_row) break;
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
        auto row8 = [&](size_t row, float* f) {
            const float4 lo = *reinterpret_cast<const float4*>(p.partials + row * p.d + c * 8);
            const float4 hi = *reinterpret_cast<const float4*>(p.partials + row * p.d + c * 8 + 4);
            f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w; f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
        };
        // every row of the sum is requested before the first is used (up to eight routed rows at a time):
        // a block has one token's rows to itself, so what it waits for is a trip to memory, not bytes
        float sh[8];
        if (p.has_shared) row8((size_t)p.tokens * p.top_k + t, sh);
        v[k] = *reinterpret_cast<const uint4*>(a.hidden + (size_t)t * a.hidden_stride + c * 8);
        wv[k] = *reinterpret_cast<const uint4*>(a.weight + c * 8);
        if (p.has_shared) {
            const float gate = __fadd_rn(1.0f, expf(-gate_in));
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float s = p.gate_logit ? __fdiv_rn(sh[j], gate) : sh[j];
                acc[j] = __fadd_rn(acc[j], s);
            }
        }
        for (uint32_t r0 = 0; r0 < p.top_k; r0 += 8) {
            float pr[8][8], w[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) {          // slots past the last reread it and are not used
                const uint32_t rr = min(r0 + r, p.top_k - 1u);
                w[r] = f16_to_f32(p.w[(size_t)t * p.top_k + rr]);
                row8((size_t)t * p.top_k + rr, pr[r]);
            }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                if (r0 + r < p.top_k) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[j] = __fadd_rn(acc[j], __fmul_rn(w[r], pr[r][j]));
                }
            }
        }
        uint4 y16;
        uint32_t* yy = reinterpret_cast<uint32_t*>(&y16);
#pragma unroll
        for (int j = 0; j < 4; ++j) yy[j] = (uint32_t)f32_to_act<ACT>(acc[2 * j]) | ((uint32_t)f32_to_act<ACT>(acc[2 * j + 1]) << 16);
        if (p.y) *reinterpret_cast<uint4*>((uint16_t*)p.y + (size_t)t * p.y_stride + c * 8) = y16;
        uint32_t* vv = reinterpret_cast<uint32_t*>(&v[k]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a0, a1, b0, b1;
            act2_to_f32<ACT>(vv[j], a0, a1);
            act2_to_f32<ACT>(yy[j], b0, b1);
            vv[j] = (uint32_t)f32_to_act<ACT>(__fadd_rn(a0, b0)) | ((uint32_t)f32_to_act<ACT>(__fadd_rn(a1, b1)) << 16);
        }
        reinterpret_cast<uint4*>(post_raw)[c] = v[k];
        *reinterpret_cast<uint4*>(a.hidden + (size_t)t * a.hidden_stride + c * 8) = v[k];
    }
    __syncthreads();
    // the stated order: lane l over the elements l, l + 64, ...; every wave for itself
    float sum = 0.0f;
    for (uint32_t i0 = lane; i0 < p.d; i0 += 512) {
        uint16_t e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = i0 + 64 * j < p.d ? post_raw[i0 + 64 * j] : (uint16_t)0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (i0 + 64 * j >= p.d) break;
            const float x = act_to_f32<ACT>(e[j]);
            sum = fmaf(x, x, sum);
        }
    }
    const float inv = rms_inverse(rms_wave_sum(sum), p.d, a.eps);
#pragma unroll
    for (int k = 0; k < ROUTER_PRE_PIECES; ++k) {
        const uint32_t c = threadIdx.x + 256 * k;
        if (c >= per_row) break;
        const uint32_t* vv = reinterpret_cast<const uint32_t*>(&v[k]);
        const uint32_t* ww = reinterpret_cast<const uint32_t*>(&wv[k]);
        uint4 o;
        uint32_t* oo = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a0, a1, w0, w1;
            act2_to_f32<ACT>(vv[j], a0, a1);
            act2_to_f32<ACT_BF16>(ww[j], w0, w1);
            oo[j] = (uint32_t)f32_to_act<ACT>(__fmul_rn(__fmul_rn(a0, inv), w0)) |
                    ((uint32_t)f32_to_act<ACT>(__fmul_rn(__fmul_rn(a1, inv), w1)) << 16);
        }
        *reinterpret_cast<uint4*>(a.normed + (size_t)t * a.normed_stride + c * 8) = o;
    }
}

// ---- small decode batches: three launches instead of five ---------------------------------
// With a handful of tokens the step is bound by its chain of dependent launches, not by bytes.
// (1) expert_rows_routed: the gate/up launch selects for itself.  Every wave repeats its token's
// top-k from the logits (256 floats; the same routine as the select kernels, so the same indices)
// and takes the expert of its block's slot from it; grid.y = token, a block's entry is (token,
// slot) with slot top_k = the shared expert.  The first block of a token stores the routes.
// Tokens that share an expert read it once each (from L2 after the first).
struct RoutedStats {
    uint32_t* stats;           // optional: [0] = entries, [1] = distinct routed experts of the step
    int has_shared;
};

template <int ACT, int BITS, int SEG, int NCH, int RPI, int ITERS>
__global__ __launch_bounds__(256) void expert_rows_routed(RowsParams p, SelectParams sel, RoutedStats rs) {
    extern __shared__ uint4 rows_lds[];
    const uint32_t slot = blockIdx.x / p.blocks_per_entry, rb = blockIdx.x % p.blocks_per_entry;
    const uint32_t t = blockIdx.y;
    const int lane = threadIdx.x & 63;
    WorkEntry we;
    we.pair_count = 1;
    we.reserved = t;
    if (slot < sel.top_k) {
        float score;
        uint32_t idx;
        select_topk_core(sel, t, lane, score, idx);
        if (blockIdx.x == 0 && threadIdx.x < 64) {
            select_store_routes(sel, t, lane, score, idx);
        }
        we.expert = (uint32_t)__builtin_amdgcn_readlane((int)idx, (int)slot);
        we.pair_start = t * sel.top_k + slot;
    } else {
        we.expert = NVMAI_SLOT_FLAG | 8u;
        we.pair_start = sel.tokens * sel.top_k + t;
    }
    expert_rows_body<ACT, BITS, SEG, NCH, 1, true, false, RPI, ITERS, ROWS_DIRECT>(p, we, rb, rows_lds);
    // The caller's statistics, off the critical path: the first block counts the distinct experts
    // of the step once its rows are done (at most four tokens, tokens * top_k <= 64 indices).
    if (rs.stats && blockIdx.x == 0 && t == 0) {
        const uint32_t n = sel.tokens * sel.top_k;
        uint32_t distinct = sel.top_k;
        if (sel.tokens > 1) {
            __syncthreads();
            uint32_t* ids = reinterpret_cast<uint32_t*>(rows_lds);
            const uint32_t wave = threadIdx.x >> 6;
            if (wave < sel.tokens) {
                float score;
                uint32_t idx;
                select_topk_core(sel, wave, lane, score, idx);
                if ((uint32_t)lane < sel.top_k) ids[wave * sel.top_k + lane] = idx;
            }
            __syncthreads();
            bool first = (uint32_t)lane < n;
            for (uint32_t j = 0; j < (uint32_t)lane && (uint32_t)lane < n; ++j) first = first && ids[j] != ids[lane];
            distinct = (uint32_t)__popcll(__ballot(first));
        }
        if (threadIdx.x == 0) {
            rs.stats[0] = sel.tokens * (sel.top_k + (rs.has_shared ? 1u : 0u));
            rs.stats[1] = distinct;
        }
    }
}

// The routed experts of ONE token given as a table of blob pointers (the reference's RoutedBlobs,
// moe.metal:153-155): entry i = slot i -- or active_slots[i], skipped when it is not below top_k
// (the hit / miss split, moe.metal:685-727) -- input row 0, output row = slot.  No work list.
template <int ACT, int BITS, int SEG, int NCH, int RPI, int ITERS>
__global__ __launch_bounds__(256) void expert_rows_slots(RowsParams p, const uint32_t* active_slots, uint32_t top_k) {
    extern __shared__ uint4 rows_lds[];
    const uint32_t entry = blockIdx.x / p.blocks_per_entry, rb = blockIdx.x % p.blocks_per_entry;
    const uint32_t slot = active_slots ? active_slots[entry] : entry;
    if (slot >= top_k) return;                    // uniform per block
    WorkEntry we;
    we.expert = NVMAI_SLOT_FLAG | slot;
    we.pair_start = slot;
    we.pair_count = 1;
    we.reserved = 0;
    expert_rows_body<ACT, BITS, SEG, NCH, 1, true, false, RPI, ITERS, ROWS_DIRECT>(p, we, rb, rows_lds);
}

// (2) down_combine: the down projection of every slot of a token and the weighted sum over the
// slots in one launch.  A block owns DC_ROWS output rows of one token; its four waves share the
// slots (wave w: slots w, w + 4, ...), SEG lanes per row with one 16-byte chunk each, every load
// of a wave issued before the first use.  Plain fp32: dot = fma chain over the chunk in element
// order, acc = scale * dot + bias * sum(act), DPP sum over the row's lanes.  The slot partials
// meet in LDS and DC_ROWS threads add them exactly as combine_kernel does (shared expert first,
// then the routed slots in slot order).
constexpr int DC_ROWS = 8;
constexpr int DC_SLOTS_PER_WAVE = 3;        // top_k + shared <= 12

struct DownCombineParams {
    BlobSource src;
    int64_t wA, sA, bA;           // down projection inside the blob
    const float* acts;            // fp32 [tokens * top_k (+ tokens), n]: routed rows, then shared rows
    const uint32_t* idx;          // [tokens, top_k] pool indices; NULL: slot s reads the blob in table slot s
    const uint16_t* w;            // fp16 [tokens, top_k]
    const void* residual;         // optional activations [tokens, res_stride], added first
    uint32_t res_stride;
    const float* gate_logit;      // optional [tokens]
    int has_shared;
    uint32_t tokens, top_k, rows, n, y_stride;
    void* y;
};

// (Handing a slot's activation row to the lanes through LDS -- one fetch per wave instead of one
// per row of a load instruction -- was measured slower: 12 us against 9.6 us per launch at one
// token; the step is a chain of latencies, and the LDS round trip lengthens it.)
template <int ACT, int BITS, int SEG>
__global__ __launch_bounds__(256) void down_combine_kernel(DownCombineParams p) {
    constexpr int EPC = Chunk<BITS>::elems;
    constexpr int RPL = 64 / SEG;                 // rows per load instruction
    constexpr int PASSES = DC_ROWS / RPL;
    __shared__ float part[4 * DC_SLOTS_PER_WAVE][DC_ROWS];
    const uint32_t t = blockIdx.y, row0 = blockIdx.x * DC_ROWS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int seg_id = lane / SEG, sl = lane % SEG;
    const uint32_t n_slots = p.top_k + (p.has_shared ? 1u : 0u);
    const uint32_t groups = p.n / NVMAI_GROUP, row_bytes = p.n * BITS / 8;
    const uint32_t g = (uint32_t)sl * EPC / NVMAI_GROUP;

    // what the final sum needs, requested before everything else: lane k holds the weight of slot k
    const float wk = (uint32_t)lane < p.top_k ? f16_to_f32(p.w[(size_t)t * p.top_k + lane]) : 0.0f;
    const float gate = p.gate_logit ? p.gate_logit[t] : 0.0f;
    const float res = p.residual && wave == 0 && lane < DC_ROWS && row0 + lane < p.rows
                          ? act_to_f32<ACT>(((const uint16_t*)p.residual)[(size_t)t * p.res_stride + row0 + lane]) : 0.0f;

    uint4 q[DC_SLOTS_PER_WAVE][PASSES];
    uint16_t sc[DC_SLOTS_PER_WAVE][PASSES], bi[DC_SLOTS_PER_WAVE][PASSES];
    float a[DC_SLOTS_PER_WAVE][EPC];
#pragma unroll
    for (int j = 0; j < DC_SLOTS_PER_WAVE; ++j) {
        const uint32_t slot = wave + 4 * j;
        if (slot >= n_slots) break;               // uniform per wave
        const bool routed = slot < p.top_k;
        const uint32_t expert = !routed ? (NVMAI_SLOT_FLAG | 8u)
                                : p.idx ? p.idx[(size_t)t * p.top_k + slot] : (NVMAI_SLOT_FLAG | slot);
        const uint32_t act_row = routed ? t * p.top_k + slot : p.tokens * p.top_k + t;
        const uint8_t* blob = blob_ptr(p.src, expert);
        const uint8_t* W = blob + p.wA;
        const uint16_t* S = reinterpret_cast<const uint16_t*>(blob + p.sA);
        const uint16_t* B = reinterpret_cast<const uint16_t*>(blob + p.bA);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const uint32_t row = row0 + i * RPL + seg_id;
            const uint32_t r = row < p.rows ? row : p.rows - 1;
            q[j][i] = *reinterpret_cast<const uint4*>(W + (size_t)r * row_bytes + sl * 16);
            sc[j][i] = S[(size_t)r * groups + g];
            bi[j][i] = B[(size_t)r * groups + g];
        }
        load_x<ACT, true, EPC>(p.acts, (size_t)act_row * p.n, (uint32_t)sl * EPC, a[j]);
    }
#pragma unroll
    for (int j = 0; j < DC_SLOTS_PER_WAVE; ++j) {
        const uint32_t slot = wave + 4 * j;
        if (slot >= n_slots) break;
        const float* aj = a[j];
        float xs = 0.0f;
#pragma unroll
        for (int e = 0; e < EPC; ++e) xs += aj[e];
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            float qf[EPC];
            unpack_chunk<BITS>(q[j][i], qf);
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < EPC; ++e) dot = fmaf(qf[e], aj[e], dot);
            float acc = fmaf(bf16_to_f32(sc[j][i]), dot, bf16_to_f32(bi[j][i]) * xs);
            acc = seg_reduce_sum<SEG>(acc);
            if (seg_result_lane<SEG>(lane)) part[slot][i * RPL + seg_id] = acc;
        }
    }
    __syncthreads();
    if (wave == 0) {              // lanes below DC_ROWS own an output row each; all 64 serve the lane reads
        const uint32_t r = lane < DC_ROWS ? lane : 0;
        float acc = res;
        if (p.has_shared) {
            float s = part[p.top_k][r];
            if (p.gate_logit) s = __fdiv_rn(s, __fadd_rn(1.0f, expf(-gate)));
            acc = __fadd_rn(acc, s);
        }
        for (uint32_t k = 0; k < p.top_k; ++k)
            acc = __fadd_rn(acc, __fmul_rn(readlane_f(wk, (int)k), part[k][r]));
        if (lane < DC_ROWS && row0 + r < p.rows)
            ((uint16_t*)p.y)[(size_t)t * p.y_stride + row0 + r] = f32_to_act<ACT>(acc);
    }
}

// fp32 rows [tokens, m] -> the caller's rows with its own stride: 16-bit activations (y) and /
// or fp32 (yf).  blockIdx.y = token.
template <int ACT>
__global__ void store_rows_kernel(const float* a, void* y, float* yf, uint32_t m, uint32_t y_stride) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (i >= m) return;
    const float v = a[(size_t)t * m + i];
    if (y) ((uint16_t*)y)[(size_t)t * y_stride + i] = f32_to_act<ACT>(v);
    if (yf) yf[(size_t)t * y_stride + i] = v;
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
