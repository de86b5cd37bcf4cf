// Gated delta rule over long calls with BF16 activations: the chunk recurrence of gdn_chunk_kernels.hpp
// with everything that does not depend on the state taken out of the chain, and the chain's products on
// the 16-bit matrix instructions from operands split into two BF16 halves.
//
// With T, W, G, beta, c of a chunk as gdn_chunk_prep_kernel leaves them, and S the state the chunk finds:
//     D = T R,  R[i] = beta_i v_i - beta_i G_i (S k_i)      becomes      D = U - Kt S^T
//     U  = T diag(beta) V          (sixteen rows of dv values; no state in it)
//     Kt = T diag(beta G) K        (sixteen rows of dk values; no state in it)
// so a chunk's chain is: split S, Kt S^T, a subtraction, the state update -- one wave, sixteen state rows
// (columns of S^T), no partial sums through LDS and no barrier inside the chain.
//   * Kt is made once per (sequence, value head, chunk) by gdn_wy_prep_kernel, in fp32 on
//     v_mfma_f32_16x16x4_f32 (k is a 16-bit value, T and beta G are fp32), and stored as two BF16 halves
//     hi + lo (hi = the upper sixteen bits of the float, lo = the rest rounded: together 16 bits of
//     mantissa) in the lane order of the A operand of v_mfma_f32_16x16x32_bf16.
//   * The state stays fp32 in the accumulators of the update.  Each chunk splits it the same way:
//     hi by a byte permute; lo = S - hi by a matrix instruction with minus the identity as A operand (the
//     accumulator layout of a tile is the B-operand layout of v_mfma_f32_16x16x16_bf16, so hi is already
//     where it has to be and the subtraction is exact), then one packed conversion.
//     Kt S^T = Kt_hi S_hi + Kt_lo S_hi + Kt_hi S_lo (the lo x lo term is below 2^-16 of the product);
//     q and k are BF16 values, so S q takes two products and the update k^T (c D) two, with c D split.
//   * U and the rows y need products over the chunk's sixteen rows only; they stay on the fp32 matrix
//     instruction.
// The wave that runs the chain (wave 0) takes a chunk's operands from LDS; three more waves bring them
// there: producer w owns the chunks n with n % 3 == w, keeps two of them in flight in registers (six chunks
// ahead of the chain in all), computes U for its chunk and writes the chunk's LDS image one iteration before
// the chain reads it.  A fifth wave makes the rows y = G (S q) + W D of the chunk before: the chain leaves
// the two halves of the state it found and D in LDS, and neither S q nor the dependent products behind D
// hold it up (inside the chain's wave they were 40 % of its time: a wave issues in order, so the next chunk
// waited behind the stores of y).  One s_barrier per chunk couples the five; it is issued bare (after
// lgkmcnt(0)), so the producers' loads stay in flight across it.
#pragma once
#include <type_traits>
#include "gdn_chunk_kernels.hpp"

namespace nvmai {

struct GdnChunkWY {
    uint4 kt_hi[4][64];     // Kt, A operand of product j: lane (m = lane % 16, g = lane / 16) holds
    uint4 kt_lo[4][64];     //   Kt[m][32 j + 4 g + e], e < 4, then Kt[m][32 j + 16 + 4 g + e]
};
static_assert(sizeof(GdnChunkWY) == 8192, "layout");

struct GdnChunkKT {
    uint2 t[8][64];         // k^T, A operand of the update of tile bb: lane (i = lane % 16, g) holds k_{4 g + e}[16 bb + i]
};
static_assert(sizeof(GdnChunkKT) == 4096, "layout");

typedef __bf16 gc_b8 __attribute__((ext_vector_type(8)));
typedef __bf16 gc_b2 __attribute__((ext_vector_type(2)));
typedef float gc_f2 __attribute__((ext_vector_type(2)));
typedef uint32_t gc_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t gc_u2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ gc_f4 gc_mfma32b(gc_u4 a, gc_u4 b, gc_f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gc_b8, a), __builtin_bit_cast(gc_b8, b), c, 0, 0, 0);
}
__device__ __forceinline__ gc_f4 gc_mfma16b(gc_u2 a, gc_u2 b, gc_f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gc_s4, a), __builtin_bit_cast(gc_s4, b), c, 0, 0, 0);
}
// the upper halves of two floats as one dword (a in the low half)
__device__ __forceinline__ uint32_t gc_hi2(float a, float b) {
    return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ uint32_t gc_rne2(float a, float b) {
    const gc_f2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, gc_b2));
}
// what the upper sixteen bits leave behind, rounded to BF16
__device__ __forceinline__ uint32_t gc_lo2(float a, float b) {
    return gc_rne2(a - __uint_as_float(__float_as_uint(a) & 0xFFFF0000u), b - __uint_as_float(__float_as_uint(b) & 0xFFFF0000u));
}

// ---- per (chunk, value head, sequence): T, W and the gate vectors, then Kt in two halves, and k^T once per key head
// One wave: the preparation of gdn_chunk_kernels.hpp and, from what it leaves in LDS, the split operands.
__global__ __launch_bounds__(64) void gdn_wy_prep_kernel(GdnDeltaParams p, GdnChunkPrep* prep, GdnChunkWY* wy, GdnChunkKT* kts,
                                                        uint32_t nchunks) {
    constexpr int DK = 128;
    __shared__ GdnPrepLds l;
    __shared__ __attribute__((aligned(16))) GdnPrepKeep<DK> keep;
    __shared__ __attribute__((aligned(16))) float kt[16][DK + 4];
    gdn_chunk_prep_body<ACT_BF16, DK, true>(p, prep, nchunks, l, &keep);
    __syncthreads();
    const uint32_t lane = threadIdx.x, i16 = lane & 15u, g = lane >> 4;
    const uint32_t c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const GdnShape& sh = p.sh;
    const uint32_t ratio = sh.v_heads / sh.k_heads, hk = h / ratio;
    float Tp[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) Tp[s] = keep.Ts[i16][4 * g + s] * keep.bG[4 * g + s];
    GdnChunkKT* ko = kts + ((size_t)b * sh.k_heads + hk) * nchunks + c;
    const bool write_kt = h % ratio == 0;
#pragma unroll
    for (int bb = 0; bb < DK / 16; ++bb) {
        uint16_t raw[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) raw[s] = keep.ks[4 * g + s][16 * bb + i16];
        gc_f4 C = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s) C = gc_mfma4(Tp[s], bf16_to_f32(raw[s]), C);       // C[r] = Kt[4 g + r][16 bb + i16]
#pragma unroll
        for (int r = 0; r < 4; ++r) kt[4 * g + r][16 * bb + i16] = C[r];
        if (write_kt) ko->t[bb][lane] = uint2{(uint32_t)raw[0] | ((uint32_t)raw[1] << 16), (uint32_t)raw[2] | ((uint32_t)raw[3] << 16)};
    }
    __syncthreads();
    GdnChunkWY* wo = wy + ((size_t)b * sh.v_heads + h) * nchunks + c;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float4 a = *reinterpret_cast<const float4*>(&kt[i16][32 * j + 4 * g]);
        const float4 d = *reinterpret_cast<const float4*>(&kt[i16][32 * j + 16 + 4 * g]);
        wo->kt_hi[j][lane] = uint4{gc_hi2(a.x, a.y), gc_hi2(a.z, a.w), gc_hi2(d.x, d.y), gc_hi2(d.z, d.w)};
        wo->kt_lo[j][lane] = uint4{gc_lo2(a.x, a.y), gc_lo2(a.z, a.w), gc_lo2(d.x, d.y), gc_lo2(d.z, d.w)};
    }
}

// ---- the chunks in sequence ------------------------------------------------------------------------------
struct GdnWySlot {          // a chunk's operands for the chain, lane order throughout; two of them in turn
    uint4 kt_hi[4][64], kt_lo[4][64];
    uint2 kT[8][64];
    float4 U[64];           // U[4 g + r][dv]
    float c[16];
    float G15, pad[3];
};
struct GdnWyRowSlot {       // a chunk's operands for its rows y; three in turn (read one iteration after the chain's)
    uint4 q[4][64];         // A operand of S q: q[m][32 j + 4 g + e], then q[m][32 j + 16 + 4 g + e]
    float4 W[64];           // W[i16][4 g + s]
    float G[16];
};
struct GdnWyHand {          // what the chain hands to the wave that makes the rows; two in turn
    uint4 s_hi[4][64], s_lo[4][64];     // the state the chunk found, B operands of the products j
    float4 D[64];
};

__device__ __forceinline__ gc_u4 ld4(const uint4* p) { return *reinterpret_cast<const gc_u4*>(p); }

__device__ __forceinline__ void gdn_wy_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Waves of a block go to the four SIMDs of a compute unit in turn, and the chain should have its SIMD to itself:
// wave 0 runs the chain, wave 1 makes the rows, waves 2, 3 and 5 are the producers, wave 4 (the chain's SIMD) only
// keeps the barriers' count.  (Measured and not kept: the chain shared by two waves, half of the state columns each,
// their shares of Kt S^T exchanged through LDS at a second barrier in the middle of the iteration -- 182 against
// 153 us for 256 chunks: the barrier costs more than half of the split, the products and the update saves.)
constexpr int GDN_WY_WAVES = 6;

template <bool STATE_BF16>
__global__ __launch_bounds__(64 * GDN_WY_WAVES, 2) void gdn_wy_delta_kernel(GdnDeltaParams p, const GdnChunkPrep* prep, const GdnChunkWY* wy,
                                                          const GdnChunkKT* kts, uint32_t nchunks) {
    constexpr int DK = 128, DV = 128;
    __shared__ GdnWySlot slots[2];
    __shared__ GdnWyRowSlot rslots[3];
    __shared__ GdnWyHand hand[2];
    const uint32_t lane = threadIdx.x & 63u, i16 = lane & 15u, g = lane >> 4;
    const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);        // the same in every lane of a wave
    // 0: the chain; 1, 2, 3: producers 0, 1, 2; 4: the rows; 5: nothing
    const uint32_t role = wv == 0 ? 0u : wv == 1 ? 4u : wv == 2 ? 1u : wv == 3 ? 2u : wv == 5 ? 3u : 5u;
    const uint32_t h = blockIdx.x, b = blockIdx.y, dv = blockIdx.z * 16 + i16;
    const GdnShape& sh = p.sh;
    const uint32_t hk = h / (sh.v_heads / sh.k_heads);
    const GdnChunkPrep* pb = prep + ((size_t)b * sh.v_heads + h) * nchunks;
    const GdnChunkWY* wb = wy + ((size_t)b * sh.v_heads + h) * nchunks;
    const GdnChunkKT* kb = kts + ((size_t)b * sh.k_heads + hk) * nchunks;

    // ---- producers: a chunk in registers, then its LDS image
    // (native vector types: a struct copy from global memory is a memcpy to the compiler and pins the stage to the stack)
    struct Stage { gc_u4 kh[4], kl[4]; gc_u2 qa[4], qb[4], kT[8]; uint16_t v[4]; gc_f4 T, W, beta; float Gl, cl; };
    auto fetch = [&](uint32_t n, Stage& st) {
        n = min(n, nchunks - 1);                            // past the end: a chunk nobody reads
        const uint32_t t0 = n * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            st.kh[j] = *reinterpret_cast<const gc_u4*>(&wb[n].kt_hi[j][lane]);
            st.kl[j] = *reinterpret_cast<const gc_u4*>(&wb[n].kt_lo[j][lane]);
        }
        const uint16_t* qrow = p.conv_out + ((size_t)b * sh.rows + min(t0 + i16, sh.rows - 1)) * p.conv_stride + hk * DK;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            st.qa[j] = *reinterpret_cast<const gc_u2*>(qrow + 32 * j + 4 * g);
            st.qb[j] = *reinterpret_cast<const gc_u2*>(qrow + 32 * j + 16 + 4 * g);
        }
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) st.kT[bb] = *reinterpret_cast<const gc_u2*>(&kb[n].t[bb][lane]);
#pragma unroll
        for (int s = 0; s < 4; ++s)
            st.v[s] = p.conv_out[((size_t)b * sh.rows + min(t0 + 4 * g + s, sh.rows - 1)) * p.conv_stride + 2 * sh.k_heads * DK + h * DV + dv];
        const GdnChunkPrep* pc = pb + n;
        st.T = *reinterpret_cast<const gc_f4*>(&pc->T[i16][4 * g]);
        st.W = *reinterpret_cast<const gc_f4*>(&pc->W[i16][4 * g]);
        st.beta = *reinterpret_cast<const gc_f4*>(&pc->beta[4 * g]);
        st.Gl = pc->G[i16];
        st.cl = pc->c[i16];
    };
    auto publish = [&](uint32_t n, const Stage& st, GdnWySlot& sl) {
        GdnWyRowSlot& rs = rslots[n % 3u];
        const uint32_t keep = n * 16 + i16 < sh.rows ? 0xFFFFFFFFu : 0u;      // q rows past the end are zero
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<gc_u4*>(&sl.kt_hi[j][lane]) = st.kh[j];
            *reinterpret_cast<gc_u4*>(&sl.kt_lo[j][lane]) = st.kl[j];
            *reinterpret_cast<gc_u4*>(&rs.q[j][lane]) = gc_u4{st.qa[j].x & keep, st.qa[j].y & keep, st.qb[j].x & keep, st.qb[j].y & keep};
        }
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) *reinterpret_cast<gc_u2*>(&sl.kT[bb][lane]) = st.kT[bb];
        // U = T (beta v): contraction index m = 4 g + s (rows past the end hold beta = 0)
        gc_f4 U = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s) U = gc_mfma4(st.T[s], st.beta[s] * bf16_to_f32(st.v[s]), U);
        *reinterpret_cast<gc_f4*>(&sl.U[lane]) = U;
        *reinterpret_cast<gc_f4*>(&rs.W[lane]) = st.W;
        if (lane < 16) { rs.G[lane] = st.Gl; sl.c[lane] = st.cl; }
        if (lane == 15) sl.G15 = st.Gl;
    };

    // ---- the chain: S^T[dk = 16 bb + 4 g + r][dv] in acc[bb][r]
    const size_t sbase = (((size_t)b * sh.v_heads + h) * DV + dv) * DK + 4 * g;
    gc_f4 acc[8];
    gc_u2 negI;                                             // minus the identity as the A operand of a 16 x 16 x 16 product
    {
        uint32_t e[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) e[k] = 4 * g + k == i16 ? 0xBF80u : 0u;
        negI = gc_u2{e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
    }
    if (role == 0) {
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) {
            if (STATE_BF16) {
                const uint2 x = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.state) + sbase + 16 * bb);
                acc[bb] = gc_f4{bf16_to_f32((uint16_t)(x.x & 0xFFFFu)), bf16_to_f32((uint16_t)(x.x >> 16)),
                                bf16_to_f32((uint16_t)(x.y & 0xFFFFu)), bf16_to_f32((uint16_t)(x.y >> 16))};
            } else {
                const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.state) + sbase + 16 * bb);
                acc[bb] = gc_f4{x.x, x.y, x.z, x.w};
            }
        }
    }
    auto consume = [&](const GdnWySlot& sl, GdnWyHand& hd) {
        // every operand of the chunk is requested before the first product (the reads cannot start before the
        // barrier, and a read issued where it is used leaves its latency on the chain)
        gc_u4 kth[4], ktl[4];
        gc_u2 kTv[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) kth[j] = ld4(&sl.kt_hi[j][lane]);
        const gc_f4 U = *reinterpret_cast<const gc_f4*>(&sl.U[lane]);
        const gc_f4 c4 = *reinterpret_cast<const gc_f4*>(&sl.c[4 * g]);
        const float G15 = sl.G15;
#pragma unroll
        for (int j = 0; j < 4; ++j) ktl[j] = ld4(&sl.kt_lo[j][lane]);
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) kTv[bb] = *reinterpret_cast<const gc_u2*>(&sl.kT[bb][lane]);
        __builtin_amdgcn_sched_barrier(0);
        // the state in two halves, in B-operand order
        gc_u2 hi[8], lo[8];
        gc_f4 rest[8];
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) hi[bb] = gc_u2{gc_hi2(acc[bb][0], acc[bb][1]), gc_hi2(acc[bb][2], acc[bb][3])};
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) rest[bb] = gc_mfma16b(negI, hi[bb], acc[bb]);
        // the accumulators are free from here to the update: the decay of the chunk goes in now
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) acc[bb] *= G15;
        gc_f4 P0 = {0.0f, 0.0f, 0.0f, 0.0f}, P1 = P0, P2 = P0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const gc_u4 Bh = gc_u4{hi[2 * j].x, hi[2 * j].y, hi[2 * j + 1].x, hi[2 * j + 1].y};
            P0 = gc_mfma32b(kth[j], Bh, P0);
            P1 = gc_mfma32b(ktl[j], Bh, P1);
            *reinterpret_cast<gc_u4*>(&hd.s_hi[j][lane]) = Bh;
        }
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) lo[bb] = gc_u2{gc_rne2(rest[bb][0], rest[bb][1]), gc_rne2(rest[bb][2], rest[bb][3])};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const gc_u4 Bl = gc_u4{lo[2 * j].x, lo[2 * j].y, lo[2 * j + 1].x, lo[2 * j + 1].y};
            P2 = gc_mfma32b(kth[j], Bl, P2);
            *reinterpret_cast<gc_u4*>(&hd.s_lo[j][lane]) = Bl;
        }
        // D = U - Kt S^T; the update takes c D in two halves
        const gc_f4 D = {U.x - (P0[0] + P1[0] + P2[0]), U.y - (P0[1] + P1[1] + P2[1]), U.z - (P0[2] + P1[2] + P2[2]),
                         U.w - (P0[3] + P1[3] + P2[3])};
        const float cD[4] = {c4.x * D[0], c4.y * D[1], c4.z * D[2], c4.w * D[3]};
        const gc_u2 cDh = gc_u2{gc_hi2(cD[0], cD[1]), gc_hi2(cD[2], cD[3])};
        const gc_u2 cDl = gc_u2{gc_lo2(cD[0], cD[1]), gc_lo2(cD[2], cD[3])};
        // one 32-deep product per tile: contraction slots e < 4 of a lane group are (row 4 g + e, upper half of
        // c D), slots 4 .. 7 the same rows with the lower half, so k^T stands twice in the A operand
        const gc_u4 cD2 = gc_u4{cDh.x, cDh.y, cDl.x, cDl.y};
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) acc[bb] = gc_mfma32b(gc_u4{kTv[bb].x, kTv[bb].y, kTv[bb].x, kTv[bb].y}, cD2, acc[bb]);
        *reinterpret_cast<gc_f4*>(&hd.D[lane]) = D;
    };
    // the rows of chunk c from what the chain left behind: y = G (S q) + W D
    uint16_t* const yrow = p.out + ((size_t)b * sh.rows + 4 * g) * p.out_stride + h * DV + dv;
    auto rows_of = [&](uint32_t c, const GdnWyRowSlot& rs, const GdnWyHand& hd) {
        const uint32_t t0 = c * 16;
        gc_f4 Q0 = {0.0f, 0.0f, 0.0f, 0.0f}, Q1 = Q0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const gc_u4 qv = ld4(&rs.q[j][lane]);
            Q0 = gc_mfma32b(qv, ld4(&hd.s_hi[j][lane]), Q0);
            Q1 = gc_mfma32b(qv, ld4(&hd.s_lo[j][lane]), Q1);
        }
        const gc_f4 G4 = *reinterpret_cast<const gc_f4*>(&rs.G[4 * g]);
        const gc_f4 Wf = *reinterpret_cast<const gc_f4*>(&rs.W[lane]);
        const gc_f4 D = *reinterpret_cast<const gc_f4*>(&hd.D[lane]);
        gc_f4 Y = {G4.x * (Q0[0] + Q1[0]), G4.y * (Q0[1] + Q1[1]), G4.z * (Q0[2] + Q1[2]), G4.w * (Q0[3] + Q1[3])};
#pragma unroll
        for (int s = 0; s < 4; ++s) Y = gc_mfma4(Wf[s], D[s], Y);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (t0 + 4 * g + r < sh.rows) yrow[(size_t)(t0 + r) * p.out_stride] = f32_to_bf16(Y[r]);
    };

    // Iteration i: the chain works on chunk i (slot i % 2) while producer (i + 1) % 3 writes chunk i + 1 into the
    // other slot and requests chunk i + 7, and the fifth wave makes the rows of chunk i - 1.  Every wave meets the
    // others at one barrier before the first iteration and at one at the end of each iteration, nchunks + 1 in
    // all; each kind of wave runs a loop of its own so that the state, the producers' stages and the rows'
    // operands do not share registers.  A producer's loop is written around its own chunks -- stage A, three
    // barriers, stage B, three barriers -- so that the compiler sees which stage's loads are the older ones and
    // waits for those only.
    if (role == 5) {
        for (uint32_t i = 0; i <= nchunks; ++i) gdn_wy_barrier();
        return;
    }
    if (role == 4) {
        gdn_wy_barrier();
        for (uint32_t i = 0; i < nchunks; ++i) {
            if (i != 0) rows_of(i - 1, rslots[(i - 1) % 3u], hand[(i - 1) & 1u]);
            gdn_wy_barrier();
        }
        rows_of(nchunks - 1, rslots[(nchunks - 1) % 3u], hand[(nchunks - 1) & 1u]);
        return;
    }
    if (role != 0) {
        Stage sA, sB;
        const uint32_t pw = role - 1;
        uint32_t first = pw;
        if (pw == 0) {
            fetch(0, sB);
            fetch(3, sA);
            publish(0, sB, slots[0]);
            fetch(6, sB);
            first = 3;
        } else {
            fetch(pw, sA);
            fetch(pw + 3, sB);
        }
        gdn_wy_barrier();
        uint32_t passed = 0;                                // barriers of the loop behind this wave
        // chunk n may be written once iteration n - 2 is over, and has to be there when iteration n - 1 ends
        // (both exits inside the body: the back edge then always follows stage B's requests; a stage's next
        // chunk is requested behind the barrier that hands its chunk over, so the chain does not wait for the
        // issue of three dozen loads)
        for (uint32_t n = first;; n += 6) {
            if (n >= nchunks) break;
            for (; passed + 1 < n; ++passed) gdn_wy_barrier();
            publish(n, sA, slots[n & 1u]);
            gdn_wy_barrier();
            ++passed;
            fetch(n + 6, sA);
            if (n + 3 >= nchunks) break;
            for (; passed + 1 < n + 3; ++passed) gdn_wy_barrier();
            publish(n + 3, sB, slots[(n + 3) & 1u]);
            gdn_wy_barrier();
            ++passed;
            fetch(n + 9, sB);
        }
        for (; passed < nchunks; ++passed) gdn_wy_barrier();
        return;
    }
    gdn_wy_barrier();
    for (uint32_t i = 0; i < nchunks; ++i) {
        consume(slots[i & 1u], hand[i & 1u]);
        gdn_wy_barrier();
    }
    {
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) {
            if (STATE_BF16) {
                const uint32_t lo = (uint32_t)f32_to_bf16(acc[bb][0]) | ((uint32_t)f32_to_bf16(acc[bb][1]) << 16);
                const uint32_t hi = (uint32_t)f32_to_bf16(acc[bb][2]) | ((uint32_t)f32_to_bf16(acc[bb][3]) << 16);
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.state) + sbase + 16 * bb) = uint2{lo, hi};
            } else {
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.state) + sbase + 16 * bb) =
                    float4{acc[bb][0], acc[bb][1], acc[bb][2], acc[bb][3]};
            }
        }
    }
}

}  // namespace nvmai
