// Causal attention of a prefill chunk over a quantized K/V cache (prefill.metal:709-830), for gfx950, in two
// launches: the chunk's key range is dequantized ONCE into fp16 scratch -- K rows as they are, V transposed --
// and a flash-attention kernel then runs plain fp16 products on it.  Every key row of a chunk is read by
// hundreds of query blocks, so taking the codes apart once per row instead of once per (row, query block) is
// what pays here (in a decode step every row is read once, and the kernels of attn_kernels.hpp multiply the
// codes themselves).  head_dim 256, up to 16 q heads per kv head.
#pragma once

#include "attn_kernels.hpp"

namespace nvmai {

// ---- K/V rows [lo0, lo0 + ntok) -> kd [kv head][token][256] fp16, vt [kv head][256][token] fp16 (the tokens of
// every 32-token tile permuted, see below) ---------------------------------------------------------------------
// One block per (32 tokens, kv head).  w = code * scale + bias in fp32, rounded once to fp16
// (attention.metal:89-117 dequantizes the same way; the fp16 rounding is 2^-11 relative, the 8-bit
// quantization step it sits on 2^-8 of the group's range).  Rows at or past `hi` become zeros; with a ring the
// row of key p is p % ring.
struct AttnDequantParams {
    const uint8_t* k;
    const uint8_t* v;
    KvFormat f;
    uint32_t ring;
    uint32_t lo0, hi, ntok;          // ntok a multiple of 32
    uint32_t kv_heads;
    uint16_t* kd;
    uint16_t* vt;
};

// fp16 of x, saturating: a row whose scale and bias reach past the fp16 range (values of 1e5 and more) stays finite.
__device__ __forceinline__ uint16_t attn_f16_sat(float x) { return f32_to_f16(fminf(fmaxf(x, -65504.0f), 65504.0f)); }

__device__ __forceinline__ void attn_dequant32(const uint8_t* row, const KvFormat& f, uint32_t e0, bool live, bool vec, uint16_t* out) {
    if (!live) {
#pragma unroll
        for (int e = 0; e < 32; ++e) out[e] = 0;
        return;
    }
    if (vec && f.bits != 16) {
        const uint32_t groups = (f.elements + 63) / 64;
        const uint16_t* meta = reinterpret_cast<const uint16_t*>(row + f.value_bytes);
        const float s = f16_to_f32(meta[e0 / 64]), b = f16_to_f32(meta[groups + e0 / 64]);
        if (f.bits == 8) {
            const uint4 a = *reinterpret_cast<const uint4*>(row + e0), c = *reinterpret_cast<const uint4*>(row + e0 + 16);
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
#pragma unroll
            for (int e = 0; e < 32; ++e) out[e] = attn_f16_sat(fmaf((float)((w[e >> 2] >> (8 * (e & 3))) & 0xFFu), s, b));
        } else {
            const uint4 a = *reinterpret_cast<const uint4*>(row + e0 / 2);
            const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
            for (int e = 0; e < 32; ++e) out[e] = attn_f16_sat(fmaf((float)((w[e >> 3] >> (4 * (e & 7))) & 0xFu), s, b));
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 32; ++e) out[e] = attn_f16_sat(kv_load(row, f, e0 + e));
}

__global__ __launch_bounds__(256) void attn_prefill_dequant_kernel(AttnDequantParams p) {
    __shared__ uint16_t tile[32][ATTN_HD + 8];
    const uint32_t tok0 = blockIdx.x * 32, kvh = blockIdx.y;
    const uint32_t tl = threadIdx.x >> 3, d0 = (threadIdx.x & 7u) * 32;
    const uint32_t pos = p.lo0 + tok0 + tl;
    const bool live = pos < p.hi;
    const uint32_t rix = p.ring ? pos % p.ring : pos;
    const bool vec = (p.f.stride % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.k) | reinterpret_cast<uintptr_t>(p.v)) & 15u) == 0;
    const uint32_t e0 = kvh * ATTN_HD + d0;
    uint16_t h[32];
    attn_dequant32(p.k + (size_t)rix * p.f.stride, p.f, e0, live, vec, h);
    uint4* kdst = reinterpret_cast<uint4*>(p.kd + ((size_t)kvh * p.ntok + tok0 + tl) * ATTN_HD + d0);
#pragma unroll
    for (int q = 0; q < 4; ++q)
        kdst[q] = uint4{(uint32_t)h[8 * q] | ((uint32_t)h[8 * q + 1] << 16), (uint32_t)h[8 * q + 2] | ((uint32_t)h[8 * q + 3] << 16),
                        (uint32_t)h[8 * q + 4] | ((uint32_t)h[8 * q + 5] << 16), (uint32_t)h[8 * q + 6] | ((uint32_t)h[8 * q + 7] << 16)};
    attn_dequant32(p.v + (size_t)rix * p.f.stride, p.f, e0, live, vec, h);
#pragma unroll
    for (int e = 0; e < 32; ++e) tile[tl][d0 + e] = h[e];
    __syncthreads();
    const uint32_t dim = threadIdx.x;                     // one dim, the 32 tokens of the block
    // tokens of the tile in the order the flash-attention kernel multiplies them: piece r (16 bytes) holds
    // the tokens 4r .. 4r+3 and 16+4r .. 16+4r+3, the eight contraction slots of lane quarter r
    uint16_t c[32];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
#pragma unroll
        for (int j = 0; j < 8; ++j) c[rr * 8 + j] = tile[(j >> 2) * 16 + 4 * rr + (j & 3)][dim];
    uint4* vdst = reinterpret_cast<uint4*>(p.vt + ((size_t)kvh * ATTN_HD + dim) * p.ntok + tok0);
#pragma unroll
    for (int q = 0; q < 4; ++q)
        vdst[q] = uint4{(uint32_t)c[8 * q] | ((uint32_t)c[8 * q + 1] << 16), (uint32_t)c[8 * q + 2] | ((uint32_t)c[8 * q + 3] << 16),
                        (uint32_t)c[8 * q + 4] | ((uint32_t)c[8 * q + 5] << 16), (uint32_t)c[8 * q + 6] | ((uint32_t)c[8 * q + 7] << 16)};
}

// ---- flash attention over the fp16 scratch -------------------------------------------------------------------
// One block of NW waves (4 or 8) per (kv head, NW * 16 / qpk consecutive query tokens): wave w owns sixteen score columns -- 16 / qpk
// query tokens x the qpk heads of the group -- for the whole key range; the waves share every 32-token
// K / V tile, which reaches LDS without passing through registers (buffer_load ... lds), the next tile while
// this one is multiplied: one barrier per tile.
//   S[tokens, columns] = K . Q^T    A = K rows from LDS, B = q * (scale log2 e) as fp16, in registers
//   O[columns, dims]   = P . V      A = the probabilities where the scores left them (the accumulator layout of
//                                   S is the A-operand layout of this product when the contraction index of a
//                                   lane's eight slots runs over tokens 4r..4r+3 of both 16-token tiles),
//                                   B = V^T rows from LDS
// Lane roles (i = lane % 16, r = lane / 16):
//   K operand (tile, ks): token 16 tile + i, dims 32 ks + 8 r .. + 8;  Q operand: column i, the same dims
//   S accumulators: column i, tokens 4r .. 4r+3 of the tile
//   V operand (g, n): dim 64 g + 16 n + i, tokens {4r..4r+3, 16+4r..16+4r+3} = piece r of the row;  O accumulators: that dim, columns 4r..4r+3
// LDS: a K tile is [token][32 chunks of 16 bytes], chunk c of token t in slot c ^ (t % 16); a V^T tile is
// [dim][4 pieces of eight tokens], piece c of dim d in slot c ^ sigma(d): both operand reads touch every bank once.
constexpr uint32_t ATTN_FA_KTILE = 32 * ATTN_HD * 2;      // bytes
constexpr float ATTN_FA_LAZY = 6.0f;                        // see the softmax of attn_prefill_fa_kernel
constexpr uint32_t ATTN_FA_MIN_BLOCKS = 256;              // blocks below which the one-launch kernels are taken
// Slot swizzle of a V^T row (rows of 64 bytes, sixteen lanes reading piece r of sixteen consecutive dims): chosen by
// measurement -- a wave's 16-byte reads at slot r ^ ((d / 2) % 4) run at the rate of a linear read (1.9 ns per
// wave-read and compute unit with eight waves reading), unswizzled or swizzled by (d / 4) % 4 at half of it.
__device__ __forceinline__ uint32_t attn_fa_vsigma(uint32_t d) { return (d >> 1) & 3u; }

// Maximum over the four lane quarters (lanes l, l ^ 16, l ^ 32, l ^ 48) by the two row-swap instructions of this
// target: a swap hands every lane its partner's value in one of its two results, so the maximum of the two is the
// pairwise maximum in every lane -- vector instructions of a few cycles where a bpermute is a trip through LDS,
// and this maximum heads the dependency chain of every tile.
__device__ __forceinline__ float attn_fa_max_quarters(float v) {
    typedef unsigned u2_t __attribute__((ext_vector_type(2)));
    const u2_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a.x), __uint_as_float(a.y));
    const u2_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b.x), __uint_as_float(b.y));
}

template <int ACT, int NW>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void attn_prefill_fa_kernel(AttnParams p, const uint16_t* kd, const uint16_t* vt, uint32_t ntok,
                                                                 uint32_t lo0) {
    __shared__ __attribute__((aligned(16))) uint8_t k0s[ATTN_FA_KTILE];
    __shared__ __attribute__((aligned(16))) uint8_t k1s[ATTN_FA_KTILE];
    __shared__ __attribute__((aligned(16))) uint8_t v0s[ATTN_FA_KTILE];
    __shared__ __attribute__((aligned(16))) uint8_t v1s[ATTN_FA_KTILE];
    constexpr int LPW = 16 / NW;                                   // load instructions per wave, tile and array
    __shared__ float bc_all[64 * NW];
    __shared__ uint32_t rng[2 * NW];
    // the tiles are written by load instructions only; a store that never runs keeps the optimizer from treating
    // them as never written (head_dim 0 is rejected by the entry point)
    if (p.head_dim == 0) { k0s[threadIdx.x] = 0; k1s[threadIdx.x] = 0; v0s[threadIdx.x] = 0; v1s[threadIdx.x] = 0; }
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, r = lane >> 4;
    float* bc = bc_all + wave * 64;
    const uint32_t qpk = p.num_q_heads / p.num_kv_heads;           // 1, 2, 4, 8 or 16
    const uint32_t tpw = 16u / qpk, tpb = (uint32_t)NW * tpw;                // query tokens per wave, per block
    const uint32_t n_qb = (p.batch + tpb - 1) / tpb;
    const uint32_t kvh = blockIdx.x % p.num_kv_heads;
    const uint32_t qb = n_qb - 1u - blockIdx.x / p.num_kv_heads;   // the longest key ranges start first
    const uint32_t b_w = qb * tpb + wave * tpw;                    // first query token of this wave
    const bool live = b_w + (uint32_t)i / qpk < p.batch;
    const uint32_t my_b = live ? b_w + (uint32_t)i / qpk : 0u, my_h = kvh * qpk + (uint32_t)i % qpk;
    uint32_t lo_i = 0u, hi_i = 0u;
    if (live) attn_range(p, my_b, lo_i, hi_i);
    // key range of the wave (union and intersection over its live columns) and of the block
    uint32_t wlo = live ? lo_i : 0xFFFFFFFFu, whi = live ? hi_i : 0u, ilo = live ? lo_i : 0u, ihi = live ? hi_i : 0xFFFFFFFFu;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        wlo = min(wlo, shfl_xor_u(wlo, off)); whi = max(whi, shfl_xor_u(whi, off));
        ilo = max(ilo, shfl_xor_u(ilo, off)); ihi = min(ihi, shfl_xor_u(ihi, off));
    }
    wlo = __builtin_amdgcn_readfirstlane(wlo); whi = __builtin_amdgcn_readfirstlane(whi);
    ilo = __builtin_amdgcn_readfirstlane(ilo); ihi = __builtin_amdgcn_readfirstlane(ihi);
    if (lane == 0) { rng[wave] = wlo; rng[NW + wave] = whi; }
    __syncthreads();
    uint32_t blo = rng[0], bhi = rng[NW];
#pragma unroll
    for (int w = 1; w < NW; ++w) { blo = min(blo, rng[w]); bhi = max(bhi, rng[NW + w]); }
    // tiles of the scratch: tile t holds the keys lo0 + 32 t .. + 32
    const uint32_t t_first = blo < bhi ? (blo - lo0) / 32u : 0u, t_end = blo < bhi ? (bhi - lo0 + 31u) / 32u : 0u;

    // ---- Q: column i, scaled by scale * log2(e) so that the scores are exponents of two, as fp16
    uint4 qop[8];
    {
        const uint16_t* qh = (const uint16_t*)p.q + (size_t)my_b * p.q_stride + (size_t)my_h * ATTN_HD;
        const float qs = p.scale * 1.44269504088896340736f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const uint4 raw = live ? *reinterpret_cast<const uint4*>(qh + 32 * ks + 8 * r) : uint4{0u, 0u, 0u, 0u};
            float f[8];
            act2_to_f32<ACT>(raw.x, f[0], f[1]); act2_to_f32<ACT>(raw.y, f[2], f[3]);
            act2_to_f32<ACT>(raw.z, f[4], f[5]); act2_to_f32<ACT>(raw.w, f[6], f[7]);
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (uint32_t)attn_f16_sat(f[2 * e] * qs) | ((uint32_t)attn_f16_sat(f[2 * e + 1] * qs) << 16);
            qop[ks] = uint4{w[0], w[1], w[2], w[3]};
        }
    }

    // ---- tile loads: the sixteen 1 KB pieces of the K tile (two tokens each) and of the V^T tile (sixteen dims each)
    // are dealt over the waves
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(kd), 0, (int)((size_t)p.num_kv_heads * ntok * ATTN_HD * 2), 0x00020000);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(vt), 0, (int)((size_t)p.num_kv_heads * ntok * ATTN_HD * 2), 0x00020000);
    uint32_t k_off[LPW], v_off[LPW];
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const uint32_t tok = 2u * ((uint32_t)LPW * wave + j) + ((uint32_t)lane >> 5), slot = (uint32_t)lane & 31u;
        k_off[j] = ((kvh * ntok + tok) * ATTN_HD) * 2u + ((slot ^ (tok & 15u)) * 16u);
        const uint32_t dim = 16u * ((uint32_t)LPW * wave + j) + ((uint32_t)lane >> 2), s16 = (uint32_t)lane & 3u;
        v_off[j] = ((kvh * ATTN_HD + dim) * ntok) * 2u + ((s16 ^ attn_fa_vsigma(dim)) * 16u);
    }
    auto issue_tile = [&](uint32_t t, uint8_t* ks, uint8_t* vs) {
#if defined(__HIP_DEVICE_COMPILE__)     // the host pass rejects the 16-byte form of the load
#pragma unroll
        for (int j = 0; j < LPW; ++j) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(krsrc, (__attribute__((address_space(3))) void*)(ks + (LPW * wave + j) * 1024), 16,
                                                     k_off[j], t * (32u * ATTN_HD * 2u), 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(vrsrc, (__attribute__((address_space(3))) void*)(vs + (LPW * wave + j) * 1024), 16,
                                                     v_off[j], t * 64u, 0, 0);
        }
#endif
    };

    f4_t oacc[4][4];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int n = 0; n < 4; ++n) oacc[g][n] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -1e30f, d_run = 0.0f;                             // column i; d over this lane's tokens only

    // operand addresses inside a tile
    uint32_t ka[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) ka[ks] = (uint32_t)i * 512u + ((((uint32_t)(4 * ks + r)) ^ (uint32_t)i) & 31u) * 16u;
    const uint32_t va = (uint32_t)i * 64u + (((uint32_t)r ^ attn_fa_vsigma((uint32_t)i)) * 16u);   // dim 64 g + 16 n + i, piece r
    auto slot_tok = [&](int t) { return (uint32_t)((t >> 2) * 16 + 4 * r + (t & 3)); };

    auto compute = [&](uint32_t t, const uint8_t* ks_, const uint8_t* vs_) {
        const uint32_t pos0 = lo0 + 32u * t;
        if (pos0 >= whi || pos0 + 32u <= wlo) return;               // wave-uniform: no key of this wave's columns
        // four accumulators (even and odd steps of the head dimension for each half of the tile), so that a
        // product never waits for the one before it
        f4_t sacc4[4] = {f4_t{0.0f, 0.0f, 0.0f, 0.0f}, f4_t{0.0f, 0.0f, 0.0f, 0.0f}, f4_t{0.0f, 0.0f, 0.0f, 0.0f}, f4_t{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            H8 a0, a1, b;
            const uint4 w0 = *reinterpret_cast<const uint4*>(ks_ + ka[ks]);
            const uint4 w1 = *reinterpret_cast<const uint4*>(ks_ + ka[ks] + 16 * 512);
            a0.u[0] = w0.x; a0.u[1] = w0.y; a0.u[2] = w0.z; a0.u[3] = w0.w;
            a1.u[0] = w1.x; a1.u[1] = w1.y; a1.u[2] = w1.z; a1.u[3] = w1.w;
            b.u[0] = qop[ks].x; b.u[1] = qop[ks].y; b.u[2] = qop[ks].z; b.u[3] = qop[ks].w;
            sacc4[2 * (ks & 1)] = mfma16(a0, b, sacc4[2 * (ks & 1)]);
            sacc4[2 * (ks & 1) + 1] = mfma16(a1, b, sacc4[2 * (ks & 1) + 1]);
        }
        const f4_t sacc[2] = {sacc4[0] + sacc4[2], sacc4[1] + sacc4[3]};
        float sv[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) sv[s] = sacc[s >> 2][s & 3];
        if (!(pos0 >= ilo && pos0 + 32u <= ihi)) {                  // wave-uniform: some column masks some key of the tile
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const uint32_t pos = pos0 + slot_tok(s);
                sv[s] = (pos >= lo_i && pos < hi_i) ? sv[s] : -INFINITY;
            }
        }
        // ---- online softmax for column i (its tokens are spread over the four lane quarters)
        float mx = sv[0];
#pragma unroll
        for (int s = 1; s < 8; ++s) mx = fmaxf(mx, sv[s]);
        mx = attn_fa_max_quarters(mx);
        // The reference point of the column's exponentials moves only when the maximum has grown by more than
        // ATTN_FA_LAZY (the probabilities then reach 2^ATTN_FA_LAZY at most, well inside fp16 and exact in the
        // final quotient): after the first tiles O is hardly ever rescaled.
        // (m_run starts at a finite -1e30: a column that has seen no key yet needs no case of its own, the
        // exponentials of its masked scores are 2^-inf = 0 and alpha is 2^0)
        const float m_new = mx > m_run + ATTN_FA_LAZY ? mx : m_run;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        float pe[8], psum = 0.0f;
#pragma unroll
        for (int s = 0; s < 8; ++s) { pe[s] = __builtin_amdgcn_exp2f(sv[s] - m_new); psum += pe[s]; }
        d_run = d_run * alpha + psum;
        m_run = m_new;
        typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
        typedef float f2_t __attribute__((ext_vector_type(2)));
        H8 pop;
#pragma unroll
        for (int w = 0; w < 4; ++w) pop.u[w] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{pe[2 * w], pe[2 * w + 1]}, h2_t));
        // ---- O of columns 4r .. 4r+3 follows their running maxima
        if (__any(alpha != 1.0f)) {
            if (r == 0) bc[i] = alpha;                              // column-indexed broadcast through LDS
            __builtin_amdgcn_wave_barrier();
            const float4 al = *reinterpret_cast<const float4*>(bc + 4 * r);
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int n = 0; n < 4; ++n) {
                    oacc[g][n][0] *= al.x; oacc[g][n][1] *= al.y; oacc[g][n][2] *= al.z; oacc[g][n][3] *= al.w;
                }
        }
        // ---- O += P . V
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                const uint4 x = *reinterpret_cast<const uint4*>(vs_ + (64 * g + 16 * n) * 64 + va);
                H8 bop;
                bop.u[0] = x.x; bop.u[1] = x.y; bop.u[2] = x.z; bop.u[3] = x.w;
                oacc[g][n] = mfma16(pop, bop, oacc[g][n]);
            }
    };

    // ---- the tiles in order, two per trip so that the stage arrays are named at compile time
    if (t_first < t_end) issue_tile(t_first, k0s, v0s);
    for (uint32_t t = t_first; t < t_end; t += 2) {
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0): this wave's part of tile t has landed
        __syncthreads();                                            // everybody's has; nobody still reads the other stage
        if (t + 1 < t_end) issue_tile(t + 1, k1s, v1s);
        compute(t, k0s, v0s);
        if (t + 1 >= t_end) break;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (t + 2 < t_end) issue_tile(t + 2, k0s, v0s);
        compute(t + 1, k1s, v1s);
    }

    // ---- finish: d over the four quarters, O / d, rows out through LDS in 16-byte pieces
    d_run += shfl_xor_f(d_run, 16);
    d_run += shfl_xor_f(d_run, 32);
    if (r == 0) bc[i] = d_run;
    __builtin_amdgcn_wave_barrier();
    const float4 d4 = *reinterpret_cast<const float4*>(bc + 4 * r);
    __builtin_amdgcn_wave_barrier();
    const float dd[4] = {d4.x, d4.y, d4.z, d4.w};
    __syncthreads();                                                // every wave is through with the tiles
    uint8_t* const stage = (wave >> 1) == 0 ? k0s : (wave >> 1) == 1 ? k1s : (wave >> 1) == 2 ? v0s : v1s;
    uint16_t* orow = reinterpret_cast<uint16_t*>(stage + (wave & 1) * 8192);   // [16 columns][256]
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int c = 0; c < 4; ++c)
                orow[(4 * r + c) * ATTN_HD + 64 * g + 16 * n + i] = f32_to_act<ACT>(dd[c] > 0.0f ? oacc[g][n][c] / dd[c] : 0.0f);
    __builtin_amdgcn_wave_barrier();
    // 16 columns x 512 bytes = 512 pieces of 16 bytes: eight per lane
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const uint32_t piece = (uint32_t)q * 64u + (uint32_t)lane, c = piece >> 5, at = (piece & 31u) * 8u;
        const uint32_t tok = b_w + c / qpk;
        if (tok >= p.batch) continue;
        const uint4 val = *reinterpret_cast<const uint4*>(orow + c * ATTN_HD + at);
        *reinterpret_cast<uint4*>((uint16_t*)p.out + (size_t)tok * p.out_stride + (size_t)(kvh * qpk + c % qpk) * ATTN_HD + at) = val;
    }
}

}  // namespace nvmai
