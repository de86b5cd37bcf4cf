// Affine 4 / 8-bit group-64 matrix times 5 .. 32 input rows on the matrix cores, for gfx950: the
// product a decode step of a small batch needs for its projections and its LM head
// (dequant_int4.metal:93-215 and dequant_int8.metal's GEMV kernels, issued once per token there).
// The row engine streams the matrix once per four inputs; here a block reads its 64 rows once for
// up to 32 inputs.
//
// Arithmetic: the factored form of the reference (nvmai_kernels.h:19-21)
//     y[row, tok] = sum_g  s[row, g] * (sum_{k in g} q[row, k] x[tok, k])  +  b[row, g] * (sum_{k in g} x[tok, k])
// with the inner sums on v_mfma_f32_16x16x32_f16: the codes themselves are the A operand, read as
// fp16 subnormals (code * 2^-24; the matrix cores take subnormal inputs exactly), the inputs the
// B operand -- each input row scaled by a power of two so that its largest magnitude lies in
// [1024, 2048) and rounded to fp16, as the row engine stages them.  One accumulator per group of
// 64, so that scale and bias are applied exactly per group, in fp32.
//
// Block = 16 WR matrix rows x all inputs: WR of the four waves stand side by side on the rows (16
// each), the 4 / WR waves behind each other share out the stages of K and add their partial
// results through LDS at the end -- a matrix of a few thousand rows still gives every compute
// unit a block (WR = 1), a large one keeps the inputs' staging cost per row low (WR = 4).
// Codes, scales and biases travel
// memory -> LDS without passing through registers (buffer_load ... lds), two stages of 512 codes
// per row in flight per wave; the 16-byte chunks of a row are XOR-swizzled by the row so that the
// operand reads of sixteen rows touch every bank once.  The inputs are staged once per panel of K
// (2048 elements for up to 16 inputs, 1024 for up to 32) as fp16 rows 16 bytes longer than the
// panel, which spreads the sixteen tokens of an operand read over the banks.
// Lane roles (i = lane % 16, r = lane / 16):
//   A operand, group g, half h:  row i, codes 64 g + 16 r + 8 h .. + 8
//   B operand:                   input i (of the tile), the same k
//   accumulators:                input i, rows 4 r .. 4 r + 3
#pragma once

#include "common.hpp"

namespace nvmai {

struct GemvMfmaParams {
    const uint8_t* w;          // [m, n * bits / 8] codes
    const uint16_t* s;         // BF16 [m, n / 64]
    const uint16_t* b;
    const uint16_t* x;         // [n_tokens, x_stride] activations
    uint32_t x_stride, n_tokens;
    uint32_t m, n;
    uint16_t* y;               // [n_tokens, y_stride] activations, or null
    float* y_f32;              // [n_tokens, y_stride] fp32, or null
    uint32_t y_stride;
};

typedef _Float16 gm_h8_t __attribute__((ext_vector_type(8)));
typedef float gm_f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t gm_u4_t __attribute__((ext_vector_type(4)));
union GmH8 { gm_h8_t v; uint32_t u[4]; uint4 q; };

// s_waitcnt operand: at most n vector-memory loads still in flight, the other counters free.
constexpr int gm_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

// Power of two that maps amax into [1024, 2048), and its inverse; 1 for zero, tiny or non-finite.
__device__ __forceinline__ void gm_pow2_scale(float amax, float& sc, float& isc) {
    const uint32_t e = (__float_as_uint(amax) >> 23) & 0xFFu;
    if (e < 24u || e > 254u) { sc = 1.0f; isc = 1.0f; return; }
    sc = __uint_as_float((264u - e) << 23);
    isc = __uint_as_float((e - 10u) << 23);
}

constexpr uint32_t GM_STAGE_CODES = 512;        // codes of a row per stage: 8 groups

// NW = waves per block (4 or 8): eight halve what a wave has to stage and to multiply, which is
// what a projection of a few thousand rows -- one block per compute unit at most -- is short of.
template <int ACT, int BITS, int TT, int WR, int NW>
__global__ __launch_bounds__(64 * NW) void gemv_mfma_kernel(GemvMfmaParams p) {
    constexpr int KW = NW / WR;                          // waves sharing out the stages of K
    constexpr uint32_t KP = 2048 / TT;                   // elements of an input panel
    constexpr uint32_t XROW = KP * 2 + 16;               // bytes of a staged input row
    constexpr uint32_t NTOK = 16 * TT;
    constexpr uint32_t SB = GM_STAGE_CODES * BITS / 8;   // bytes of one row's codes in a stage
    constexpr uint32_t WREG = 16 * SB;                   // a wave's 16 rows of a stage
    constexpr int CPR = SB / 16;                         // 16-byte chunks per row: 16 or 32
    constexpr int RPI = 64 / CPR;                        // rows per load instruction: 4 or 2
    constexpr int NLD = 16 / RPI;                        // code loads per stage: 4 or 8
    constexpr int N_LOADS = NLD + 2;                     // + scales + biases
    constexpr uint32_t GPP = KP / 64;                    // groups per panel
    __shared__ __attribute__((aligned(16))) uint8_t x_s[NTOK * XROW];
    __shared__ __attribute__((aligned(16))) uint8_t wa[NW * WREG];
    __shared__ __attribute__((aligned(16))) uint8_t wb[NW * WREG];
    __shared__ __attribute__((aligned(16))) uint8_t ma[NW * 512];    // per wave: 16 rows x 16 B scales | 16 x 16 B biases
    __shared__ __attribute__((aligned(16))) uint8_t mb[NW * 512];
    __shared__ __attribute__((aligned(16))) float xsum_s[NTOK * GPP];
    __shared__ float isc_s[NTOK];
    // the stage arrays are written by load instructions only; a store that never runs keeps the
    // optimizer from treating them as never written (n = 0 is rejected by the host)
    if (p.n == 0) { wa[threadIdx.x] = 0; wb[threadIdx.x] = 0; ma[threadIdx.x] = 0; mb[threadIdx.x] = 0; }

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, r = lane >> 4;
    const int wave_r = wave % WR, wave_k = wave / WR;
    const uint32_t row0 = blockIdx.x * (16 * WR) + wave_r * 16;
    const uint32_t groups = p.n / 64, row_bytes = p.n * BITS / 8;
    const uint32_t n_stages = p.n / GM_STAGE_CODES;
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.w), 0, (int)(p.m * row_bytes), 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.s), 0, (int)(p.m * groups * 2), 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t brsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.b), 0, (int)(p.m * groups * 2), 0x00020000);

    // ---- weight stages: lane l of load j fetches chunk (l % CPR) ^ row of row j RPI + l / CPR,
    // which lands in slot l % CPR of that row; rows past the matrix reread its last row
    const uint32_t ld_row = lane / CPR, ld_slot = lane % CPR;
    uint32_t ld_off[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const uint32_t row = j * RPI + ld_row;
        const uint32_t grow = min(row0 + row, p.m - 1);
        ld_off[j] = grow * row_bytes + ((ld_slot ^ (row & 15u)) * 16u);
    }
    // scales / biases of a stage: 16 rows x 16 bytes, one dword per lane (every lane takes part:
    // a load under a lane mask would sit in a block of its own, and the compiler then loses track of
    // which LDS array the loads in flight write)
    [[maybe_unused]] const uint32_t meta_off = (min(row0 + (uint32_t)lane / 4u, p.m - 1) * groups) * 2u + ((uint32_t)lane % 4u) * 4u;
    uint8_t* const wa_w = wa + wave * WREG;
    uint8_t* const wb_w = wb + wave * WREG;
    uint8_t* const ma_w = ma + wave * 512;
    uint8_t* const mb_w = mb + wave * 512;
    auto issue_stage = [&](uint32_t st, uint8_t* wdst, uint8_t* mdst) {
#if defined(__HIP_DEVICE_COMPILE__)     // the host pass rejects the 16-byte form of the load and then drops the kernel's stub
#pragma unroll
        for (int j = 0; j < NLD; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, (__attribute__((address_space(3))) void*)(wdst + j * 1024), 16,
                                                     ld_off[j], st * SB, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(srsrc, (__attribute__((address_space(3))) void*)mdst, 4, meta_off,
                                                 st * 16u, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(brsrc, (__attribute__((address_space(3))) void*)(mdst + 256), 4,
                                                 meta_off, st * 16u, 0, 0);
#endif
    };
    // this wave's stages: wave_k, wave_k + KW, ...; its j-th one lands in the A arrays for even j
    const uint32_t n_my = (uint32_t)wave_k < n_stages ? (n_stages - wave_k + KW - 1) / KW : 0u;
    if (n_my > 0) issue_stage(wave_k, wa_w, ma_w);
    if (n_my > 1) issue_stage(wave_k + KW, wb_w, mb_w);

    // ---- inputs of one panel: a wave converts whole rows (tokens wave, wave + NW, ...)
    auto stage_inputs = [&](uint32_t k0) {
        constexpr int CH = KP / 512;                         // 16-byte pieces per lane and row
        const uint32_t kp_len = min(KP, p.n - k0);
        // every load of the wave's rows is issued before the first is used
        constexpr int TPW = NTOK / NW;                       // rows per wave
        uint4 raw_all[TPW][CH];
#pragma unroll
        for (int q = 0; q < TPW; ++q) {
            const uint32_t t = wave + NW * q;
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const uint32_t e = (c * 64 + lane) * 8;
                raw_all[q][c] = (t < p.n_tokens && e < kp_len)
                                    ? *reinterpret_cast<const uint4*>(p.x + (size_t)t * p.x_stride + k0 + e)
                                    : uint4{0u, 0u, 0u, 0u};
            }
        }
#pragma unroll
        for (int q = 0; q < TPW; ++q) {
            const uint32_t t = wave + NW * q;
            const uint4* raw = raw_all[q];
            float v[CH][8];
            float amax = 0.0f;
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                act2_to_f32<ACT>(raw[c].x, v[c][0], v[c][1]); act2_to_f32<ACT>(raw[c].y, v[c][2], v[c][3]);
                act2_to_f32<ACT>(raw[c].z, v[c][4], v[c][5]); act2_to_f32<ACT>(raw[c].w, v[c][6], v[c][7]);
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[c][j]));
            }
            amax = wave_max_f32(amax);
            float sc, isc;
            gm_pow2_scale(amax, sc, isc);
            if (lane == 0) isc_s[t] = isc;
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                uint16_t hb[8];
                float sum = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    hb[j] = f32_to_f16(v[c][j] * sc);
                    sum += f16_to_f32(hb[j]);
                }
                sum = seg_reduce_sum<8>(sum);                // the 64 elements of a group sit in 8 lanes
                if (seg_result_lane<8>(lane)) xsum_s[t * GPP + (c * 64 + lane) / 8] = sum;
                uint4 o;
                if (BITS == 8) {                             // natural order, as the code bytes unpack
                    o.x = hb[0] | ((uint32_t)hb[1] << 16); o.y = hb[2] | ((uint32_t)hb[3] << 16);
                    o.z = hb[4] | ((uint32_t)hb[5] << 16); o.w = hb[6] | ((uint32_t)hb[7] << 16);
                } else {                                     // pairs (j, j + 4), as a dword's nibbles unpack
                    o.x = hb[0] | ((uint32_t)hb[4] << 16); o.y = hb[1] | ((uint32_t)hb[5] << 16);
                    o.z = hb[2] | ((uint32_t)hb[6] << 16); o.w = hb[3] | ((uint32_t)hb[7] << 16);
                }
                *reinterpret_cast<uint4*>(x_s + t * XROW + (c * 64 + lane) * 16) = o;
            }
        }
        __syncthreads();
    };

    gm_f4_t total[TT];
    float ys[TT][4], yb[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        total[tt] = gm_f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < 4; ++t) { ys[tt][t] = 0.0f; yb[tt][t] = 0.0f; }
    }
    // fold a finished panel into the totals with that panel's input scales
    auto close_panel = [&]() {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const float isc = isc_s[tt * 16 + i];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                total[tt][t] += fmaf(ys[tt][t], 16777216.0f, yb[tt][t]) * isc;
                ys[tt][t] = 0.0f; yb[tt][t] = 0.0f;
            }
        }
    };

    // ---- one stage: 8 groups of this wave's 16 rows against the staged inputs
    auto compute_stage = [&](uint32_t st, const uint8_t* wsrc, const uint8_t* msrc) {
        const uint32_t gp0 = (st * 8u) % GPP;                    // first group of the stage inside the panel
        // scales and biases of rows 4 r .. 4 r + 3: 8 groups each, 16 bytes
        // (read like the codes below, with instructions the compiler does not track)
        gm_u4_t sc4[4], bi4[4];
        {
            [[maybe_unused]] const uint32_t maddr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)msrc + r * 64;
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile(
                "ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:16\n ds_read_b128 %2, %8 offset:32\n ds_read_b128 %3, %8 offset:48\n"
                "ds_read_b128 %4, %8 offset:256\n ds_read_b128 %5, %8 offset:272\n ds_read_b128 %6, %8 offset:288\n ds_read_b128 %7, %8 offset:304\n"
                "s_waitcnt lgkmcnt(0)"
                : "=&v"(sc4[0]), "=&v"(sc4[1]), "=&v"(sc4[2]), "=&v"(sc4[3]), "=&v"(bi4[0]), "=&v"(bi4[1]), "=&v"(bi4[2]), "=&v"(bi4[3])
                : "v"(maddr)
                : "memory");
#endif
        }
        float xs[TT][8];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const float4 a = *reinterpret_cast<const float4*>(xsum_s + (tt * 16 + i) * GPP + gp0);
            const float4 b = *reinterpret_cast<const float4*>(xsum_s + (tt * 16 + i) * GPP + gp0 + 4);
            xs[tt][0] = a.x; xs[tt][1] = a.y; xs[tt][2] = a.z; xs[tt][3] = a.w;
            xs[tt][4] = b.x; xs[tt][5] = b.y; xs[tt][6] = b.z; xs[tt][7] = b.w;
        }
        // The codes of the stage's eight groups, read with instructions the compiler does not see
        // as LDS reads: for reads of one code array it waits for the loads in flight into the
        // other one as well, which would leave nothing in flight during a stage.  The waits that
        // are needed are the explicit ones around this call.
        const uint32_t wrow = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)wsrc +
                              (i / RPI) * 1024 + (i % RPI) * (CPR * 16);
        uint32_t ca[8];
#pragma unroll
        for (int g = 0; g < 8; ++g)
            ca[g] = BITS == 8 ? wrow + ((uint32_t)(4 * g + r) ^ (uint32_t)i) * 16
                              : wrow + ((uint32_t)(2 * g + (r >> 1)) ^ (uint32_t)i) * 16 + (r & 1) * 8;
        gm_u4_t c8[8];
        uint64_t c4[8];
        if (BITS == 8) {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile(
                "ds_read_b128 %0, %8\n ds_read_b128 %1, %9\n ds_read_b128 %2, %10\n ds_read_b128 %3, %11\n"
                "ds_read_b128 %4, %12\n ds_read_b128 %5, %13\n ds_read_b128 %6, %14\n ds_read_b128 %7, %15\n"
                "s_waitcnt lgkmcnt(0)"
                : "=&v"(c8[0]), "=&v"(c8[1]), "=&v"(c8[2]), "=&v"(c8[3]), "=&v"(c8[4]), "=&v"(c8[5]), "=&v"(c8[6]), "=&v"(c8[7])
                : "v"(ca[0]), "v"(ca[1]), "v"(ca[2]), "v"(ca[3]), "v"(ca[4]), "v"(ca[5]), "v"(ca[6]), "v"(ca[7])
                : "memory");
#endif
        } else {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile(
                "ds_read_b64 %0, %8\n ds_read_b64 %1, %9\n ds_read_b64 %2, %10\n ds_read_b64 %3, %11\n"
                "ds_read_b64 %4, %12\n ds_read_b64 %5, %13\n ds_read_b64 %6, %14\n ds_read_b64 %7, %15\n"
                "s_waitcnt lgkmcnt(0)"
                : "=&v"(c4[0]), "=&v"(c4[1]), "=&v"(c4[2]), "=&v"(c4[3]), "=&v"(c4[4]), "=&v"(c4[5]), "=&v"(c4[6]), "=&v"(c4[7])
                : "v"(ca[0]), "v"(ca[1]), "v"(ca[2]), "v"(ca[3]), "v"(ca[4]), "v"(ca[5]), "v"(ca[6]), "v"(ca[7])
                : "memory");
#endif
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            uint32_t kw[4];
            if (BITS == 8) {
                kw[0] = c8[g][0]; kw[1] = c8[g][1]; kw[2] = c8[g][2]; kw[3] = c8[g][3];
            } else {
                kw[0] = (uint32_t)c4[g]; kw[1] = (uint32_t)(c4[g] >> 32);
            }
            gm_f4_t sacc[TT];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                GmH8 a;
                if (BITS == 8) {
                    const uint32_t w0 = kw[2 * h], w1 = kw[2 * h + 1];
                    a.u[0] = __builtin_amdgcn_perm(w0, w0, 0x0C050C04u);      // [c0, 0, c1, 0]: two fp16 subnormals
                    a.u[1] = __builtin_amdgcn_perm(w0, w0, 0x0C070C06u);
                    a.u[2] = __builtin_amdgcn_perm(w1, w1, 0x0C050C04u);
                    a.u[3] = __builtin_amdgcn_perm(w1, w1, 0x0C070C06u);
                } else {
                    const uint32_t w = kw[h];
#pragma unroll
                    for (int j = 0; j < 4; ++j) a.u[j] = (w >> (4 * j)) & 0x000F000Fu;
                }
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    GmH8 b;
                    b.q = *reinterpret_cast<const uint4*>(x_s + (tt * 16 + i) * XROW + ((gp0 + g) * 64 + 16 * r + 8 * h) * 2);
                    sacc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, h == 0 ? gm_f4_t{0.0f, 0.0f, 0.0f, 0.0f} : sacc[tt], 0, 0, 0);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t sw = sc4[t][g >> 1], bw = bi4[t][g >> 1];
                const float sc = (g & 1) ? __uint_as_float(sw & 0xFFFF0000u) : __uint_as_float(sw << 16);
                const float bi = (g & 1) ? __uint_as_float(bw & 0xFFFF0000u) : __uint_as_float(bw << 16);
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    ys[tt][t] = fmaf(sc, sacc[tt][t], ys[tt][t]);
                    yb[tt][t] = fmaf(bi, xs[tt][g], yb[tt][t]);
                }
            }
        }
    };

    // Panels of inputs outside, this wave's stages of the panel inside.  The inner loop holds no
    // loads but the stage loads, and its waits are the explicit ones.
    constexpr uint32_t SPP = KP / GM_STAGE_CODES;                // stages per panel
    uint32_t j = 0;                                              // index into this wave's stages
    for (uint32_t k0 = 0, panel = 0; k0 < p.n; k0 += KP, ++panel) {
        if (k0 != 0) {
            close_panel();
            __syncthreads();                                     // every wave is through with the old panel
        }
        stage_inputs(k0);
        while (j < n_my && (wave_k + j * KW) / SPP == panel) {   // wave-uniform
            const uint32_t st = wave_k + j * KW;
            if (j + 1 < n_my) __builtin_amdgcn_s_waitcnt(gm_vmcnt(N_LOADS)); else __builtin_amdgcn_s_waitcnt(gm_vmcnt(0));
            if ((j & 1u) == 0) {
                compute_stage(st, wa_w, ma_w);
                __builtin_amdgcn_s_waitcnt(0xC07F);              // lgkmcnt(0): every read of the stage has returned
                if (j + 2 < n_my) issue_stage(st + 2 * KW, wa_w, ma_w);
            } else {
                compute_stage(st, wb_w, mb_w);
                __builtin_amdgcn_s_waitcnt(0xC07F);
                if (j + 2 < n_my) issue_stage(st + 2 * KW, wb_w, mb_w);
            }
            ++j;
        }
    }
    close_panel();

    // ---- the waves that shared out K add up, in a fixed order, in the wave with wave_k = 0
    if (KW > 1) {
        __syncthreads();                                         // the input rows are no longer read
        float* red = reinterpret_cast<float*>(x_s);              // [wave][TT * 4][64 lanes]
        if (wave_k != 0) {
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                for (int t = 0; t < 4; ++t) red[(wave * TT * 4 + tt * 4 + t) * 64 + lane] = total[tt][t];
        }
        __syncthreads();
        if (wave_k != 0) return;
#pragma unroll
        for (int k = 1; k < KW; ++k)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                for (int t = 0; t < 4; ++t) total[tt][t] += red[((wave_r + k * WR) * TT * 4 + tt * 4 + t) * 64 + lane];
    }

    // ---- results: input i of each tile, rows 4 r .. 4 r + 3 of this wave
    const uint32_t rbase = row0 + 4 * r;
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const uint32_t tok = tt * 16 + i;
        if (tok >= p.n_tokens || rbase >= p.m) continue;
        if (p.y_f32) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (rbase + t < p.m) p.y_f32[(size_t)tok * p.y_stride + rbase + t] = total[tt][t];
        }
        if (p.y) {
            uint16_t* dst = p.y + (size_t)tok * p.y_stride + rbase;
            if (rbase + 3 < p.m && (reinterpret_cast<uintptr_t>(dst) & 7u) == 0) {
                uint2 o;
                o.x = f32_to_act<ACT>(total[tt][0]) | ((uint32_t)f32_to_act<ACT>(total[tt][1]) << 16);
                o.y = f32_to_act<ACT>(total[tt][2]) | ((uint32_t)f32_to_act<ACT>(total[tt][3]) << 16);
                *reinterpret_cast<uint2*>(dst) = o;
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (rbase + t < p.m) dst[t] = f32_to_act<ACT>(total[tt][t]);
            }
        }
    }
}

}  // namespace nvmai
