// Gated delta rule over long calls, sixteen rows at a time on the matrix cores (gfx950, wave64).
//
// Row by row the rule is  S_i = g_i S_{i-1} + d_i k_i^T,  d_i = beta_i (v_i - g_i S_{i-1} k_i),
// y_i = S_i q_i  (gdn.metal:368-642).  Over a chunk of sixteen rows, with G_i = g_0 .. g_i and S the
// state the chunk finds:
//     (I + L) D = R,   L[i][m] = beta_i (G_i / G_m) (k_m . k_i)  (m < i),
//                      R[i]    = beta_i v_i - beta_i G_i (S k_i)
//     y_i   = G_i (S q_i) + sum_{m <= i} W[i][m] d_m,   W[i][m] = (G_i / G_m) (k_m . q_i)
//     S_end = G_15 S + sum_m (G_15 / G_m) d_m k_m^T
// T = (I + L)^-1 and W depend on the chunk's k, q and gates only, not on the state: one kernel
// computes them for every (sequence, head, chunk) at once -- the two Gram matrices on the 16-bit
// matrix instruction (k and q are 16-bit values, so the products are exact), the 16 x 16
// triangular solve in fp32 by sixteen lanes.  What is left in sequence is five small matrix
// products per chunk, S k, S q, T R, W D and the state update, all on v_mfma_f32_16x16x4_f32: fp32
// operands, so nothing is rounded on the way and the result differs from the row-by-row kernels
// by summation order only.  One wave owns sixteen state rows (columns of S^T): the state stays in
// the accumulator registers of the update, and the accumulator layout of one product is the B
// operand layout of the next when the contraction index is taken as 4 (lane / 16) + step, so
// nothing is transposed or moved between lanes.
#pragma once
#include "gdn_kernels.hpp"

namespace nvmai {

struct GdnChunkPrep {
    float T[16][16];        // (I + L)^-1
    float W[16][16];        // (G_i / G_m) (k_m . q_i), m <= i
    float G[16];            // G_i
    float bG[16];           // beta_i G_i
    float beta[16];
    float c[16];            // G_15 / G_i
};
static_assert(sizeof(GdnChunkPrep) == 2304, "layout");

typedef float gc_f4 __attribute__((ext_vector_type(4)));
typedef short gc_s4 __attribute__((ext_vector_type(4)));
typedef _Float16 gc_h4 __attribute__((ext_vector_type(4)));

template <int ACT>
__device__ __forceinline__ gc_f4 gc_mfma16(uint2 a, uint2 b, gc_f4 c) {
    if (ACT == ACT_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gc_s4, a), __builtin_bit_cast(gc_s4, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(gc_h4, a), __builtin_bit_cast(gc_h4, b), c, 0, 0, 0);
}

__device__ __forceinline__ gc_f4 gc_mfma4(float a, float b, gc_f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// ---- per (chunk, head, sequence): T, W and the gate vectors ----------------------------------------
// One wave.  Lane (i16 = lane % 16, g = lane / 16).  The work is a function of its own so that the kernel which
// goes on to the split operands of gdn_wy_kernels.hpp can run it first: with KEEP it leaves the chunk's k rows
// (dead rows zero), T and beta G in the LDS arrays of `keep` for that kernel; the caller synchronizes.
struct GdnPrepLds {
    float xs[16], bs[16];
    float Ls[16][16];
};
template <int DK>
struct GdnPrepKeep {
    uint16_t ks[16][DK + 8];
    float Ts[16][17];
    float bG[16];
};

template <int ACT, int DK, bool KEEP>
__device__ __forceinline__ void gdn_chunk_prep_body(const GdnDeltaParams& p, GdnChunkPrep* prep, uint32_t nchunks, GdnPrepLds& l,
                                                    GdnPrepKeep<DK>* keep) {
    static_assert(DK % 16 == 0, "shape");
    float (&xs)[16] = l.xs;
    float (&bs)[16] = l.bs;
    float (&Ls)[16][16] = l.Ls;
    const uint32_t lane = threadIdx.x, i16 = lane & 15u, g = lane >> 4;
    const uint32_t c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const GdnShape& sh = p.sh;
    const uint32_t hk = h / (sh.v_heads / sh.k_heads), t0 = c * 16;
    GdnChunkPrep* out = prep + ((size_t)b * sh.v_heads + h) * nchunks + c;
    // the gates of the chunk's rows: x_i = -log g_i, beta_i; rows past the end: g = 1, beta = 0
    if (lane < 16) {
        const bool live = t0 + lane < sh.rows;
        const size_t row = (size_t)b * sh.rows + min(t0 + lane, sh.rows - 1);
        const float a = act_to_f32<ACT>(p.a_proj[row * p.ab_stride + h]), bb = act_to_f32<ACT>(p.b_proj[row * p.ab_stride + h]);
        xs[lane] = live ? expf(bf16_to_f32(p.a_log[h])) * gdn_softplus(a + bf16_to_f32(p.dt_bias[h])) : 0.0f;
        bs[lane] = live ? 1.0f / (1.0f + expf(-bb)) : 0.0f;
    }
    // k.k and q.k of the chunk's rows: A operand = rows of K (or Q), B operand = rows of K as columns
    const bool row_live = t0 + i16 < sh.rows;
    const uint16_t* base = p.conv_out + ((size_t)b * sh.rows + min(t0 + i16, sh.rows - 1)) * p.conv_stride;
    gc_f4 kk = {0.0f, 0.0f, 0.0f, 0.0f}, qk = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int st = 0; st < DK / 16; ++st) {
        uint2 kf = *reinterpret_cast<const uint2*>(base + (sh.k_heads + hk) * DK + 16 * st + 4 * g);
        uint2 qf = *reinterpret_cast<const uint2*>(base + hk * DK + 16 * st + 4 * g);
        if (!row_live) { kf = uint2{0u, 0u}; qf = uint2{0u, 0u}; }
        if (KEEP) *reinterpret_cast<uint2*>(&keep->ks[i16][16 * st + 4 * g]) = kf;
        kk = gc_mfma16<ACT>(kf, kf, kk);       // kk[r] = k_{4g+r} . k_{i16}
        qk = gc_mfma16<ACT>(qf, kf, qk);       // qk[r] = q_{4g+r} . k_{i16}
    }
    __syncthreads();
    // X_i = x_0 + .. + x_i
    float Xm = 0.0f, X15 = 0.0f;
#pragma unroll
    for (int m = 0; m < 16; ++m) {
        X15 += xs[m];
        if (m <= (int)i16) Xm = X15;
    }
    float Xi[4], Xrun = 0.0f;
#pragma unroll
    for (int m = 0; m < 16; ++m) {
        Xrun += xs[m];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (m == (int)(4 * g) + r) Xi[r] = Xrun;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t i = 4 * g + r;
        const float ratio = expf(-(Xi[r] - Xm));            // G_i / G_m, used for m <= i only
        Ls[i][i16] = i16 < i ? bs[i] * ratio * kk[r] : 0.0f;
        out->W[i][i16] = i16 <= i ? ratio * qk[r] : 0.0f;
    }
    if (lane < 16) {
        const float G = expf(-Xm);
        out->G[lane] = G;
        out->bG[lane] = bs[lane] * G;
        out->beta[lane] = bs[lane];
        out->c[lane] = expf(-(X15 - Xm));
        if (KEEP) keep->bG[lane] = bs[lane] * G;
    }
    __syncthreads();
    // column j of T by forward substitution: T[i][j] = [i == j] - sum_{m < i} L[i][m] T[m][j]
    if (lane < 16) {
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float acc = i == (int)lane ? 1.0f : 0.0f;
#pragma unroll
            for (int m = 0; m < i; ++m) acc = fmaf(-Ls[i][m], t[m], acc);
            t[i] = acc;
            out->T[i][lane] = acc;
            if (KEEP) keep->Ts[i][lane] = acc;
        }
    }
}

template <int ACT, int DK>
__global__ __launch_bounds__(64) void gdn_chunk_prep_kernel(GdnDeltaParams p, GdnChunkPrep* prep, uint32_t nchunks) {
    __shared__ GdnPrepLds l;
    gdn_chunk_prep_body<ACT, DK, false>(p, prep, nchunks, l, nullptr);
}

// ---- the chunks in sequence: one block of four waves per (head, sequence, sixteen state rows) ---------
// A chunk is a chain of products each of which waits for the one before, so the waves of a block
// share the chain's long links instead of taking chunks of their own: wave w owns the 32 columns
// dk = 32 w .. 32 w + 31 of the sixteen state rows -- acc[bb][r] = S[dv][16 (2 w + bb) + 4 g + r] for
// dv = 16 blockIdx.z + lane % 16, the accumulator layout of the state update and, with contraction
// index 4 g + step, the B operand of S k and S q.  It contracts S k and S q over its own columns,
// the four partial sums meet in LDS (added in wave order by every wave, so all four hold the same
// bits), every wave repeats the small product T R and updates its own columns; the first also makes
// the rows y = G (S q) + W D and stores them (a ninth wave that owns no columns and does only that
// was measured: 450 against 382 us per 4096 rows).
constexpr int GDN_CHUNK_WAVES = 8;

template <int ACT, int DK, int DV, bool STATE_BF16>
__global__ __launch_bounds__(64 * GDN_CHUNK_WAVES) void gdn_chunk_delta_kernel(GdnDeltaParams p, const GdnChunkPrep* prep, uint32_t nchunks) {
    constexpr int NW = GDN_CHUNK_WAVES;
    constexpr int NBW = DK / 16 / NW;                   // 16-column blocks of the state per wave
    static_assert(DK % (16 * NW) == 0 && DV % 16 == 0 && DK * 2 == 256 && (NW == 4 || NW == 8), "a row of k is sixteen 16-byte pieces; a wave stages four rows");
    __shared__ __attribute__((aligned(16))) uint16_t ks[2][16][DK];
    __shared__ __attribute__((aligned(16))) uint16_t qs[2][16][DK];
    __shared__ __attribute__((aligned(16))) float red[2][NW][64][8];     // partial S k (4) and S q (4) per lane
    const uint32_t lane = threadIdx.x & 63u, w = threadIdx.x >> 6, i16 = lane & 15u, g = lane >> 4;
    const uint32_t h = blockIdx.x, b = blockIdx.y, dv = blockIdx.z * 16 + i16;
    const GdnShape& sh = p.sh;
    const uint32_t hk = h / (sh.v_heads / sh.k_heads);
    const size_t sbase = (((size_t)b * sh.v_heads + h) * DV + dv) * DK + 16 * NBW * w + 4 * g;
    gc_f4 acc[NBW];
#pragma unroll
    for (int bb = 0; bb < NBW; ++bb) {
        if (STATE_BF16) {
            const uint2 x = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.state) + sbase + 16 * bb);
            acc[bb] = gc_f4{bf16_to_f32((uint16_t)(x.x & 0xFFFFu)), bf16_to_f32((uint16_t)(x.x >> 16)),
                            bf16_to_f32((uint16_t)(x.y & 0xFFFFu)), bf16_to_f32((uint16_t)(x.y >> 16))};
        } else {
            const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.state) + sbase + 16 * bb);
            acc[bb] = gc_f4{x.x, x.y, x.z, x.w};
        }
    }
    const GdnChunkPrep* pb = prep + ((size_t)b * sh.v_heads + h) * nchunks;
    // a chunk on its way: this wave's four of the chunk's k and q rows (lane = piece i16 of row 4 w + g),
    // this lane's v values and the chunk's T / W pieces and gate vectors.  Every load is unconditional
    // (rows past the end re-read the last row and are zeroed afterwards) so that the loads stay in
    // flight over a chunk.
    struct StageKQ { uint4 k, q; };
    struct Stage { uint16_t v[4]; float4 T, W, G, bG, beta, c; float G15; };
    auto fetch_kq = [&](uint32_t c, StageKQ& st) {
        const uint32_t t0 = c * 16;
        // four waves: wave w stages rows 4 w .. 4 w + 3 of k and of q; eight: waves 0 - 3 those of k, 4 - 7 those of q
        const uint16_t* base = p.conv_out + ((size_t)b * sh.rows + min(t0 + 4 * (w & 3u) + g, sh.rows - 1)) * p.conv_stride;
        st.k = *reinterpret_cast<const uint4*>(base + ((NW == 8 && w >= 4) ? hk : sh.k_heads + hk) * DK + i16 * 8);
        if (NW == 4) st.q = *reinterpret_cast<const uint4*>(base + hk * DK + i16 * 8);
    };
    auto fetch = [&](uint32_t c, Stage& st) {
        const uint32_t t0 = c * 16;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            st.v[r] = p.conv_out[((size_t)b * sh.rows + min(t0 + 4 * g + r, sh.rows - 1)) * p.conv_stride + 2 * sh.k_heads * DK + h * DV + dv];
        const GdnChunkPrep* pc = pb + min(c, nchunks - 1);
        st.T = *reinterpret_cast<const float4*>(&pc->T[i16][4 * g]);
        st.W = *reinterpret_cast<const float4*>(&pc->W[i16][4 * g]);
        st.G = *reinterpret_cast<const float4*>(&pc->G[4 * g]);
        st.bG = *reinterpret_cast<const float4*>(&pc->bG[4 * g]);
        st.beta = *reinterpret_cast<const float4*>(&pc->beta[4 * g]);
        st.c = *reinterpret_cast<const float4*>(&pc->c[4 * g]);
        st.G15 = pc->G[15];
    };
    auto to_lds = [&](uint32_t c, uint32_t buf, const StageKQ& st) {
        const uint32_t srow = 4 * (w & 3u) + g;
        const uint32_t keep = c * 16 + srow < sh.rows ? 0xFFFFFFFFu : 0u;
        uint16_t* first = (NW == 8 && w >= 4) ? &qs[buf][srow][i16 * 8] : &ks[buf][srow][i16 * 8];
        *reinterpret_cast<uint4*>(first) = uint4{st.k.x & keep, st.k.y & keep, st.k.z & keep, st.k.w & keep};
        if (NW == 4) *reinterpret_cast<uint4*>(&qs[buf][srow][i16 * 8]) = uint4{st.q.x & keep, st.q.y & keep, st.q.z & keep, st.q.w & keep};
    };
    float ku[NBW][4];                                    // the k values of the coming update
    // front of a chunk: this wave's share of S k and S q from the state as it is now, into red[c & 1]
    auto front = [&](uint32_t c, uint32_t buf) {
        // contraction index dk = 16 (NBW w + bb) + 4 g + s
        gc_f4 P = {0.0f, 0.0f, 0.0f, 0.0f}, Q = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int bb = 0; bb < NBW; ++bb) {
            const uint32_t col = 16 * (NBW * w + bb) + 4 * g;
            const uint2 kw = *reinterpret_cast<const uint2*>(&ks[buf][i16][col]);
            const uint2 qw = *reinterpret_cast<const uint2*>(&qs[buf][i16][col]);
            float kf[4], qf[4];
            act2_to_f32<ACT>(kw.x, kf[0], kf[1]); act2_to_f32<ACT>(kw.y, kf[2], kf[3]);
            act2_to_f32<ACT>(qw.x, qf[0], qf[1]); act2_to_f32<ACT>(qw.y, qf[2], qf[3]);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                P = gc_mfma4(kf[s], acc[bb][s], P);
                Q = gc_mfma4(qf[s], acc[bb][s], Q);
            }
        }
#pragma unroll
        for (int bb = 0; bb < NBW; ++bb)
#pragma unroll
            for (int s = 0; s < 4; ++s) ku[bb][s] = act_to_f32<ACT>(ks[buf][4 * g + s][16 * (NBW * w + bb) + i16]);
        float* mine = red[c & 1u][w][lane];
        *reinterpret_cast<float4*>(mine) = float4{P[0], P[1], P[2], P[3]};
        *reinterpret_cast<float4*>(mine + 4) = float4{Q[0], Q[1], Q[2], Q[3]};
    };
    // back of a chunk, after the barrier that follows its front: the sums, the deltas, the update, the rows
    auto back = [&](uint32_t c, const Stage& st) {
        const uint32_t t0 = c * 16;
        float Ps[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) {
            const float4 a = *reinterpret_cast<const float4*>(red[c & 1u][ww][lane]);
            Ps[0] += a.x; Ps[1] += a.y; Ps[2] += a.z; Ps[3] += a.w;
        }
        // R = beta v - beta G (S k); rows past the end hold beta = 0
        const float betav[4] = {st.beta.x, st.beta.y, st.beta.z, st.beta.w}, bGv[4] = {st.bG.x, st.bG.y, st.bG.z, st.bG.w};
        const float Gv[4] = {st.G.x, st.G.y, st.G.z, st.G.w}, cv[4] = {st.c.x, st.c.y, st.c.z, st.c.w};
        const float Tf[4] = {st.T.x, st.T.y, st.T.z, st.T.w}, Wf[4] = {st.W.x, st.W.y, st.W.z, st.W.w};
        float R[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) R[r] = betav[r] * act_to_f32<ACT>(st.v[r]) - bGv[r] * Ps[r];
        // D = T R: contraction index m = 4 g + s
        gc_f4 D = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s) D = gc_mfma4(Tf[s], R[s], D);
        // S^T <- G_15 S^T + K^T (c D), this wave's columns
        const float cD[4] = {cv[0] * D[0], cv[1] * D[1], cv[2] * D[2], cv[3] * D[3]};
#pragma unroll
        for (int bb = 0; bb < NBW; ++bb) {
            acc[bb] *= st.G15;
#pragma unroll
            for (int s = 0; s < 4; ++s) acc[bb] = gc_mfma4(ku[bb][s], cD[s], acc[bb]);
        }
        // y = G (S q) + W D, stored by the first wave
        if (w == 0) {
            float Qs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) {
                const float4 bq = *reinterpret_cast<const float4*>(red[c & 1u][ww][lane] + 4);
                Qs[0] += bq.x; Qs[1] += bq.y; Qs[2] += bq.z; Qs[3] += bq.w;
            }
            gc_f4 Y = {Gv[0] * Qs[0], Gv[1] * Qs[1], Gv[2] * Qs[2], Gv[3] * Qs[3]};
#pragma unroll
            for (int s = 0; s < 4; ++s) Y = gc_mfma4(Wf[s], D[s], Y);
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (t0 + 4 * g + r < sh.rows)
                    p.out[((size_t)b * sh.rows + t0 + 4 * g + r) * p.out_stride + h * DV + dv] = f32_to_act<ACT>(Y[r]);
        }
    };
    // One barrier per chunk: an iteration runs the back of chunk c and then, with the state just updated,
    // the front of chunk c + 1, whose k and q rows reached LDS an iteration earlier.  On their way
    // meanwhile: the k / q pieces of chunks c + 2 (stored at the end of the iteration) and c + 3, the
    // other operands of chunks c + 1 and c + 2.  Chunk c travels in kq[c % 2] and st[c % 3]; the loop is
    // unrolled by six so that both stay registers.
    StageKQ kq[2];
    Stage st[3];
    fetch_kq(0, kq[0]);
    fetch_kq(1, kq[1]);
    fetch(0, st[0]);
    fetch(1, st[1]);
    to_lds(0, 0, kq[0]);
    __syncthreads();
    front(0, 0);
    fetch_kq(2, kq[0]);
    to_lds(1, 1, kq[1]);
    __syncthreads();
    uint32_t c = 0;
#define NVMAI_GDN_CHUNK_STEP(K0, K1, A, C)              \
    fetch_kq(c + 3, kq[K1]);                            \
    fetch(c + 2, st[C]);                                \
    back(c, st[A]);                                     \
    if (c + 1 >= nchunks) break;                        \
    front(c + 1, (c + 1) & 1u);                         \
    to_lds(c + 2, c & 1u, kq[K0]);                      \
    __syncthreads();                                    \
    ++c;
    for (;;) {
        NVMAI_GDN_CHUNK_STEP(0, 1, 0, 2)
        NVMAI_GDN_CHUNK_STEP(1, 0, 1, 0)
        NVMAI_GDN_CHUNK_STEP(0, 1, 2, 1)
        NVMAI_GDN_CHUNK_STEP(1, 0, 0, 2)
        NVMAI_GDN_CHUNK_STEP(0, 1, 1, 0)
        NVMAI_GDN_CHUNK_STEP(1, 0, 2, 1)
    }
#undef NVMAI_GDN_CHUNK_STEP
#pragma unroll
    for (int bb = 0; bb < NBW; ++bb) {
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

}  // namespace nvmai
