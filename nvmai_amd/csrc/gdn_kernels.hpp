// Gated-DeltaNet linear attention for gfx950: the causal depthwise conv + SiLU with the q / k head
// norm in one kernel, the gated delta rule with the gated output norm in another.  They replace the
// reference's gdn_conv_mix_decode / _prefill, gdn_conv_tail_update, gdn_qk_norm,
// gdn_delta_step_decode / _prefill and gdn_gated_norm (gdn.metal:241-642): a decode step is rows = 1,
// a prefill chunk rows > 1 with the recurrence sequential inside the kernel, and every sequence of
// a batch has its own conv tail and recurrent state.
#pragma once

#include "common.hpp"

namespace nvmai {

constexpr float GDN_RMS_EPS = 1e-6f;        // kGdnRmsEps, gdn.metal:28
constexpr int GDN_MAX_TAPS = 8;

struct GdnShape {
    uint32_t k_heads, v_heads, dk, dv, taps;
    uint32_t rows;                          // tokens per sequence in this call (1 = decode)
    uint32_t batch;
};

// x * sigmoid(x) with the hardware's 2^x and reciprocal (about an ulp each; the result is rounded to 16 bits by every
// caller): five instructions where the library's exponential and an IEEE division take some thirty, and the conv and
// gated-norm kernels of a prompt chunk are bound by exactly these.
__device__ __forceinline__ float gdn_silu(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
}
__device__ __forceinline__ float gdn_softplus(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }

// Sum over the 256 threads of a block, result in every thread.  part: 4 floats of LDS.
__device__ __forceinline__ float gdn_block_sum(float v, float* part) {
    v = wave_sum_bcast(v);
    __syncthreads();                        // part may still be read from the previous use
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    return (part[0] + part[1]) + (part[2] + part[3]);
}

// ---- conv + SiLU + q / k norm (+ tail update) -------------------------------------------------
// Block (head segment, sequence): segments 0 .. 2 Hk - 1 are the q then the k heads (Dk channels
// each, normalised: x / rms * (1 / Dk for q, 1 / sqrt(Dk) for k), gdn.metal:386-441), segments from
// 2 Hk on the value heads (Dv channels, conv only).  A thread owns channels tid, tid + 256, ... of its
// segment for all rows of the call, reads the K - 1 tail rows of its channels once, and writes the
// new tail (the last K - 1 raw rows of [old tail | chunk], gdn.metal:309-366) when it is done: no
// other thread touches those columns.  conv_out is rounded to the activation type before the norm
// reads it, as the two kernels of the reference hand it over in 16 bits.
template <int ACT>
__global__ __launch_bounds__(256) void gdn_conv_norm_kernel(const uint16_t* qkv_raw, uint32_t qkv_stride,
                                                           uint16_t* tail, const uint16_t* conv_w,
                                                           uint16_t* conv_out, uint32_t out_stride, GdnShape sh) {
    __shared__ float part[4];
    const uint32_t seg = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const uint32_t C = 2 * sh.k_heads * sh.dk + sh.v_heads * sh.dv;
    const bool is_qk = seg < 2 * sh.k_heads;
    const uint32_t seg_len = is_qk ? sh.dk : sh.dv;
    const uint32_t base = is_qk ? seg * sh.dk : 2 * sh.k_heads * sh.dk + (seg - 2 * sh.k_heads) * sh.dv;
    const uint32_t hist = sh.taps - 1;
    uint16_t* tl = tail + (size_t)b * hist * C;
    const uint16_t* raw = qkv_raw + (size_t)b * sh.rows * qkv_stride;
    uint16_t* out = conv_out + (size_t)b * sh.rows * out_stride;
    const float scale = seg < sh.k_heads ? 1.0f / (float)sh.dk : rsqrtf((float)sh.dk);
    for (uint32_t t = 0; t < sh.rows; ++t) {
        float sumsq = 0.0f;
        for (uint32_t i = tid; i < seg_len; i += 256) {
            const uint32_t ch = base + i;
            // every tap's input and weight requested before the first product: the address is chosen, not
            // the load (a load under a condition is waited for on the spot); taps past the last reread it
            uint16_t vv[GDN_MAX_TAPS], ww[GDN_MAX_TAPS];
#pragma unroll
            for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
                const uint32_t jj = min(j, hist);
                // input row in the virtual sequence [tail rows | chunk rows]
                const int src = (int)t + (int)jj - (int)hist;
                const uint16_t* at = src >= 0 ? raw + (size_t)src * qkv_stride + ch : tl + (size_t)((int)hist + src) * C + ch;
                vv[j] = *at;
                ww[j] = conv_w[ch * sh.taps + jj];
            }
            float acc = 0.0f;
#pragma unroll
            for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j)
                if (j < sh.taps) acc = fmaf(act_to_f32<ACT>(vv[j]), bf16_to_f32(ww[j]), acc);
            const uint16_t r = f32_to_act<ACT>(gdn_silu(acc));
            out[(size_t)t * out_stride + ch] = r;
            const float x = act_to_f32<ACT>(r);
            sumsq = fmaf(x, x, sumsq);
        }
        if (is_qk) {                                      // block-uniform
            const float total = gdn_block_sum(sumsq, part);
            const float inv = rsqrtf(total / (float)sh.dk + GDN_RMS_EPS);
            for (uint32_t i = tid; i < seg_len; i += 256) {   // a thread rereads only what it wrote
                uint16_t* o = out + (size_t)t * out_stride + base + i;
                *o = f32_to_act<ACT>(act_to_f32<ACT>(*o) * inv * scale);
            }
        }
    }
    // new tail row j = virtual row rows + j - hist
    for (uint32_t i = tid; i < seg_len; i += 256) {
        const uint32_t ch = base + i;
        uint16_t keep[GDN_MAX_TAPS];
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            if (j >= hist) break;
            const int src = (int)sh.rows + (int)j - (int)hist;
            const uint16_t* at = src >= 0 ? raw + (size_t)src * qkv_stride + ch : tl + (size_t)((int)hist + src) * C + ch;
            keep[j] = *at;
        }
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            if (j >= hist) break;
            tl[(size_t)j * C + ch] = keep[j];
        }
    }
}

// ---- gated delta rule + gated output norm -------------------------------------------------------
// Per value head h with state S [Dv, Dk] (gdn.metal:10-25, 443-587):
//   g = exp(-exp(A_log[h]) * softplus(a[h] + dt_bias[h])),  beta = sigmoid(b[h])
//   S *= g;  kv = S k;  S += outer((v - kv) * beta, k);  y = S q
// then out = rmsnorm(y) * weight * silu(z) over the head's Dv outputs (gdn.metal:589-642).
// Block (value head, sequence), four waves.  Sixteen lanes own one state row (Dk / 16 elements
// each), so a wave works on four rows at once and the block on sixteen; a thread keeps its share of
// all Dv / 16 row groups in registers across the rows of the call, so a prefill chunk reads and
// writes the state once.  STATE_BF16: the state is stored in BF16 (half the bytes per token; the
// arithmetic stays fp32), else in fp32 as the reference keeps it.
struct GdnDeltaParams {
    const uint16_t* conv_out;   // [batch * rows, conv_stride]: normed q, k and conv'd v
    uint32_t conv_stride;
    const uint16_t* a_proj;     // [batch * rows, ab_stride]
    const uint16_t* b_proj;
    uint32_t ab_stride;
    const uint16_t* a_log;      // BF16 [Hv]
    const uint16_t* dt_bias;    // BF16 [Hv]
    void* state;                // [batch, Hv, Dv, Dk]
    const uint16_t* z;          // [batch * rows, z_stride]
    uint32_t z_stride;
    const uint16_t* norm_w;     // BF16 [Dv]
    uint16_t* out;              // [batch * rows, out_stride]
    uint32_t out_stride;
    GdnShape sh;
};

// VEC: the state is 16-byte aligned and DK = 128 (a lane's eight values of a state row are one or two
// 16-byte loads and stores); the host chooses.
template <int ACT, int DK, int DV, bool STATE_BF16, bool VEC = false>
__global__ __launch_bounds__(256) void gdn_delta_gated_kernel(GdnDeltaParams p) {
    constexpr int EPL = DK / 16;                // state elements per lane
    constexpr int GROUPS = DV / 16;             // sixteen rows per block pass
    static_assert(DK % 16 == 0 && DV % 16 == 0 && DV <= 256 && EPL >= 1 && EPL <= 16, "shape");
    __shared__ float y_s[DV];
    __shared__ float part[4];
    const uint32_t h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const uint32_t sub = tid & 15u, row_in_pass = tid >> 4;     // 16 rows per pass
    const GdnShape& sh = p.sh;
    const uint32_t hk = h / (sh.v_heads / sh.k_heads);
    const float exp_a = expf(bf16_to_f32(p.a_log[h]));
    const float dtb = bf16_to_f32(p.dt_bias[h]);
    const size_t state_base = (((size_t)b * sh.v_heads + h) * DV) * DK;
    float s[GROUPS][EPL];
    static_assert(!VEC || EPL == 8, "VEC needs eight state values per lane");
    constexpr bool vec = VEC;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const size_t at = state_base + (size_t)(g * 16 + row_in_pass) * DK + sub * EPL;
        if (EPL == 8 && vec) {
            if (STATE_BF16) {
                const uint4 r = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.state) + at);
                act2_to_f32<ACT_BF16>(r.x, s[g][0], s[g][1 % EPL]); act2_to_f32<ACT_BF16>(r.y, s[g][2 % EPL], s[g][3 % EPL]);
                act2_to_f32<ACT_BF16>(r.z, s[g][4 % EPL], s[g][5 % EPL]); act2_to_f32<ACT_BF16>(r.w, s[g][6 % EPL], s[g][7 % EPL]);
            } else {
                const float4 r0 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.state) + at);
                const float4 r1 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.state) + at + 4);
                s[g][0] = r0.x; s[g][1 % EPL] = r0.y; s[g][2 % EPL] = r0.z; s[g][3 % EPL] = r0.w;
                s[g][4 % EPL] = r1.x; s[g][5 % EPL] = r1.y; s[g][6 % EPL] = r1.z; s[g][7 % EPL] = r1.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                s[g][e] = STATE_BF16 ? bf16_to_f32(reinterpret_cast<const uint16_t*>(p.state)[at + e])
                                     : reinterpret_cast<const float*>(p.state)[at + e];
        }
    }
    // the norm weight of this thread's output element (threads past DV read the last one: a load under a
    // condition would be waited for on the spot, and every load in flight with it)
    const uint32_t oi = min(tid, (uint32_t)DV - 1u);
    const uint16_t nw_raw = p.norm_w[oi];
    for (uint32_t t = 0; t < sh.rows; ++t) {
        const size_t row = (size_t)b * sh.rows + t;
        const uint16_t* cq = p.conv_out + row * p.conv_stride + hk * DK + sub * EPL;
        const uint16_t* ck = cq + sh.k_heads * DK;
        const uint16_t* cv = p.conv_out + row * p.conv_stride + 2 * sh.k_heads * DK + h * DV;
        float q[EPL], k[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) { q[e] = act_to_f32<ACT>(cq[e]); k[e] = act_to_f32<ACT>(ck[e]); }
        const uint16_t z_raw = p.z[row * p.z_stride + h * DV + oi];      // requested with the row's operands, used after the barrier
        const float g_decay = expf(-exp_a * gdn_softplus(act_to_f32<ACT>(p.a_proj[row * p.ab_stride + h]) + dtb));
        const float beta = 1.0f / (1.0f + expf(-act_to_f32<ACT>(p.b_proj[row * p.ab_stride + h])));
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const uint32_t dv = g * 16 + row_in_pass;
            float kv = 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) { s[g][e] *= g_decay; kv = fmaf(s[g][e], k[e], kv); }
            kv = seg_reduce_sum<16>(kv);
            const float delta = (act_to_f32<ACT>(cv[dv]) - kv) * beta;
            float o = 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) { s[g][e] = fmaf(k[e], delta, s[g][e]); o = fmaf(s[g][e], q[e], o); }
            o = seg_reduce_sum<16>(o);
            if (sub == 0) y_s[dv] = act_to_f32<ACT>(f32_to_act<ACT>(o));     // y is handed over in 16 bits
        }
        __syncthreads();
        float sumsq = 0.0f;
        for (uint32_t i = tid; i < DV; i += 256) sumsq = fmaf(y_s[i], y_s[i], sumsq);
        const float total = gdn_block_sum(sumsq, part);
        const float inv = rsqrtf(total / (float)DV + GDN_RMS_EPS);
        if (tid < DV) {                                     // DV <= 256: one element per thread
            const float normed = y_s[tid] * inv * bf16_to_f32(nw_raw);
            const float gate = gdn_silu(act_to_f32<ACT>(z_raw));
            p.out[row * p.out_stride + h * DV + tid] = f32_to_act<ACT>(normed * gate);
        }
        __syncthreads();                                    // y_s is rewritten by the next row
    }
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const size_t at = state_base + (size_t)(g * 16 + row_in_pass) * DK + sub * EPL;
        if (EPL == 8 && vec) {
            if (STATE_BF16) {
                uint4 r;
                r.x = (uint32_t)f32_to_bf16(s[g][0]) | ((uint32_t)f32_to_bf16(s[g][1 % EPL]) << 16);
                r.y = (uint32_t)f32_to_bf16(s[g][2 % EPL]) | ((uint32_t)f32_to_bf16(s[g][3 % EPL]) << 16);
                r.z = (uint32_t)f32_to_bf16(s[g][4 % EPL]) | ((uint32_t)f32_to_bf16(s[g][5 % EPL]) << 16);
                r.w = (uint32_t)f32_to_bf16(s[g][6 % EPL]) | ((uint32_t)f32_to_bf16(s[g][7 % EPL]) << 16);
                *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.state) + at) = r;
            } else {
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.state) + at) = float4{s[g][0], s[g][1 % EPL], s[g][2 % EPL], s[g][3 % EPL]};
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.state) + at + 4) =
                    float4{s[g][4 % EPL], s[g][5 % EPL], s[g][6 % EPL], s[g][7 % EPL]};
            }
            continue;
        }
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            if (STATE_BF16) reinterpret_cast<uint16_t*>(p.state)[at + e] = f32_to_bf16(s[g][e]);
            else reinterpret_cast<float*>(p.state)[at + e] = s[g][e];
        }
    }
}


// ---- a chunk of rows: the parts that do not recur, spread over the device ---------------------------
// The conv of row t reads the raw rows t - K + 1 .. t only, and the gated output norm of row t reads
// y[t] only: with many rows per call (a prefill chunk) both run with a pair of waves per (row,
// head segment) instead of inside the sequential loops above, which leaves the recurrence itself --
// S and the rows it produces -- as the only sequential part.  The sum of squares over a segment is
// taken as in the kernels above -- channels 0..63 over the lanes of a wave, channels 64..127 the same
// way, the two sums added first: the same bits.  Segments of at most 128 channels.

// conv + SiLU + q / k norm of rows [0, rows) of every sequence; the tail is read, not written.
// A wave takes eight consecutive rows of one segment, channels lane and 64 + lane (a block four such
// groups of rows): a thread keeps the windows of its two channels in registers, so a row costs it two
// two-byte loads instead of one per tap, all sixteen in flight together, and the two halves of the sum
// of squares are the wave's own two sums -- no barrier, no LDS, and nothing orders the rows of a wave,
// so their exponentials and divisions overlap.
constexpr uint32_t GDN_CONV_ROWS_PER_BLOCK = 32;

template <int ACT>
__global__ __launch_bounds__(256) void gdn_conv_norm_rows_kernel(const uint16_t* qkv_raw, uint32_t qkv_stride,
                                                                const uint16_t* tail, const uint16_t* conv_w,
                                                                uint16_t* conv_out, uint32_t out_stride, GdnShape sh) {
    constexpr uint32_t RPW = GDN_CONV_ROWS_PER_BLOCK / 4;                   // rows per wave
    const uint32_t seg = blockIdx.x, b = blockIdx.y;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t t_first = blockIdx.z * GDN_CONV_ROWS_PER_BLOCK + wave * RPW;
    if (t_first >= sh.rows) return;                                         // uniform per wave; no barrier below
    const uint32_t C = 2 * sh.k_heads * sh.dk + sh.v_heads * sh.dv;
    const bool is_qk = seg < 2 * sh.k_heads;
    const uint32_t seg_len = is_qk ? sh.dk : sh.dv;
    const uint32_t base = is_qk ? seg * sh.dk : 2 * sh.k_heads * sh.dk + (seg - 2 * sh.k_heads) * sh.dv;
    const uint32_t hist = sh.taps - 1;
    const uint16_t* tl = tail + (size_t)b * hist * C;
    const uint16_t* raw = qkv_raw + (size_t)b * sh.rows * qkv_stride;
    bool ch_live[2];
    uint32_t ch[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        ch_live[h] = lane + 64u * h < seg_len;
        ch[h] = base + (ch_live[h] ? lane + 64u * h : 0u);
    }
    float wt[2][GDN_MAX_TAPS], pre[2][GDN_MAX_TAPS];         // weights; the hist values before the current row
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            wt[h][j] = 0.0f; pre[h][j] = 0.0f;
            if (j < sh.taps) wt[h][j] = bf16_to_f32(conv_w[ch[h] * sh.taps + j]);
            if (j < hist) {
                const int src = (int)t_first - (int)hist + (int)j;       // row src of [old tail | rows]
                pre[h][j] = act_to_f32<ACT>(src >= 0 ? raw[(size_t)src * qkv_stride + ch[h]]
                                                     : tl[(size_t)((int)hist + src) * C + ch[h]]);
            }
        }
    // rows past the end read the last row again and are not used
    uint16_t curv[2][RPW];
#pragma unroll
    for (uint32_t k = 0; k < RPW; ++k)
#pragma unroll
        for (int h = 0; h < 2; ++h) curv[h][k] = raw[(size_t)min(t_first + k, sh.rows - 1u) * qkv_stride + ch[h]];
    const float scale = seg < sh.k_heads ? 1.0f / (float)sh.dk : rsqrtf((float)sh.dk);
#pragma unroll
    for (uint32_t k = 0; k < RPW; ++k) {
        const uint32_t t = t_first + k;
        if (t >= sh.rows) break;                             // uniform
        float x[2];
        uint16_t r[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float cur = act_to_f32<ACT>(curv[h][k]);
            float acc = 0.0f;
#pragma unroll
            for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
                if (j >= sh.taps) break;
                acc = fmaf(j < hist ? pre[h][j] : cur, wt[h][j], acc);
            }
#pragma unroll
            for (uint32_t j = 0; j + 1 < GDN_MAX_TAPS; ++j) pre[h][j] = j + 1 < hist ? pre[h][j + 1] : cur;
            r[h] = 0;
            x[h] = 0.0f;
            if (ch_live[h]) {
                r[h] = f32_to_act<ACT>(gdn_silu(acc));
                x[h] = act_to_f32<ACT>(r[h]);
            }
        }
        uint16_t* o = conv_out + ((size_t)b * sh.rows + t) * out_stride;
        if (!is_qk) {                                         // block-uniform
#pragma unroll
            for (int h = 0; h < 2; ++h)
                if (ch_live[h]) o[ch[h]] = r[h];
            continue;
        }
        const float s0 = wave_sum_bcast(x[0] * x[0]), s1 = wave_sum_bcast(x[1] * x[1]);
        const float total = (s0 + s1) + (0.0f + 0.0f);
        const float inv = rsqrtf(total / (float)sh.dk + GDN_RMS_EPS);
#pragma unroll
        for (int h = 0; h < 2; ++h)
            if (ch_live[h]) o[ch[h]] = f32_to_act<ACT>(x[h] * inv * scale);
    }
}

// The same rows in 16-byte pieces, for four taps, segment lengths that are multiples of eight and rows that start at
// 16-byte boundaries: sixteen lanes take eight consecutive rows of one segment, lane j the channels 8 j .. 8 j + 7 --
// one load and one store per row and lane instead of eight, and a sixteenth of the wave-wide sums' instructions per
// channel.  Same bits: the conv sum runs over the taps in the same order, and the sum of squares is the same
// balanced tree over the channel index (neighbours first: three levels inside the lane, three across lanes 0..7 for
// channels 0..63 and across lanes 8..15 for channels 64..127, the two halves added last).
constexpr uint32_t GDN_CONV8_ROWS_PER_UNIT = 8, GDN_CONV8_ROWS_PER_BLOCK = 16 * GDN_CONV8_ROWS_PER_UNIT;

template <int ACT>
__global__ __launch_bounds__(256) void gdn_conv_norm_rows8_kernel(const uint16_t* qkv_raw, uint32_t qkv_stride,
                                                                 const uint16_t* tail, const uint16_t* conv_w,
                                                                 uint16_t* conv_out, uint32_t out_stride, GdnShape sh) {
    constexpr uint32_t RPU = GDN_CONV8_ROWS_PER_UNIT, TAPS = 4, HIST = TAPS - 1;
    const uint32_t seg = blockIdx.x, b = blockIdx.y;
    const uint32_t unit = threadIdx.x >> 4, j16 = threadIdx.x & 15u;
    const uint32_t t_first = (blockIdx.z * 16 + unit) * RPU;
    if (t_first >= sh.rows) return;                                         // uniform per sixteen lanes; no barrier below
    const uint32_t C = 2 * sh.k_heads * sh.dk + sh.v_heads * sh.dv;
    const bool is_qk = seg < 2 * sh.k_heads;
    const uint32_t seg_len = is_qk ? sh.dk : sh.dv;
    const uint32_t base = is_qk ? seg * sh.dk : 2 * sh.k_heads * sh.dk + (seg - 2 * sh.k_heads) * sh.dv;
    const bool live = 8u * j16 < seg_len;
    const uint32_t ch0 = base + (live ? 8u * j16 : 0u);
    const uint16_t* tl = tail + (size_t)b * HIST * C;
    const uint16_t* raw = qkv_raw + (size_t)b * sh.rows * qkv_stride;
    auto eight = [](const uint4& v, float* f) {
        act2_to_f32<ACT>(v.x, f[0], f[1]); act2_to_f32<ACT>(v.y, f[2], f[3]);
        act2_to_f32<ACT>(v.z, f[4], f[5]); act2_to_f32<ACT>(v.w, f[6], f[7]);
    };
    // every load of the run is requested before the first is used
    uint4 wraw[4], praw[HIST], curv[RPU];
#pragma unroll
    for (int q = 0; q < 4; ++q) wraw[q] = *reinterpret_cast<const uint4*>(conv_w + (size_t)ch0 * TAPS + 8 * q);
#pragma unroll
    for (uint32_t j = 0; j < HIST; ++j) {
        const int src = (int)t_first - (int)HIST + (int)j;                  // row src of [old tail | rows]
        praw[j] = *reinterpret_cast<const uint4*>(src >= 0 ? raw + (size_t)src * qkv_stride + ch0
                                                            : tl + (size_t)((int)HIST + src) * C + ch0);
    }
#pragma unroll
    for (uint32_t k = 0; k < RPU; ++k)                                      // rows past the end read the last row again
        curv[k] = *reinterpret_cast<const uint4*>(raw + (size_t)min(t_first + k, sh.rows - 1u) * qkv_stride + ch0);
    float wt[8][TAPS], pre[8][HIST];
    {
        const uint16_t* wh = reinterpret_cast<const uint16_t*>(wraw);      // [channel][tap]
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (uint32_t j = 0; j < TAPS; ++j) wt[c][j] = bf16_to_f32(wh[c * TAPS + j]);
#pragma unroll
        for (uint32_t j = 0; j < HIST; ++j) {
            float f[8];
            eight(praw[j], f);
#pragma unroll
            for (int c = 0; c < 8; ++c) pre[c][j] = f[c];
        }
    }
    const float scale = seg < sh.k_heads ? 1.0f / (float)sh.dk : rsqrtf((float)sh.dk);
#pragma unroll
    for (uint32_t k = 0; k < RPU; ++k) {
        const uint32_t t = t_first + k;
        if (t >= sh.rows) break;                                            // uniform per sixteen lanes
        float cur[8], x[8];
        uint16_t r[8];
        eight(curv[k], cur);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            float acc = 0.0f;
#pragma unroll
            for (uint32_t j = 0; j < TAPS; ++j) acc = fmaf(j < HIST ? pre[c][j] : cur[c], wt[c][j], acc);
#pragma unroll
            for (uint32_t j = 0; j < HIST; ++j) pre[c][j] = j + 1 < HIST ? pre[c][j + 1] : cur[c];
            r[c] = live ? f32_to_act<ACT>(gdn_silu(acc)) : (uint16_t)0;
            x[c] = live ? act_to_f32<ACT>(r[c]) : 0.0f;
        }
        uint16_t* o = conv_out + ((size_t)b * sh.rows + t) * out_stride + ch0;
        if (is_qk) {                                                        // block-uniform
            float sq = ((x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3])) +
                       ((x[4] * x[4] + x[5] * x[5]) + (x[6] * x[6] + x[7] * x[7]));
            const float total = seg_reduce_sum<16>(sq) + (0.0f + 0.0f);     // lanes 0..7, lanes 8..15, then the two halves
            const float inv = rsqrtf(total / (float)sh.dk + GDN_RMS_EPS);
#pragma unroll
            for (int c = 0; c < 8; ++c) r[c] = f32_to_act<ACT>(x[c] * inv * scale);
        }
        if (live)
            *reinterpret_cast<uint4*>(o) = uint4{(uint32_t)r[0] | ((uint32_t)r[1] << 16), (uint32_t)r[2] | ((uint32_t)r[3] << 16),
                                                 (uint32_t)r[4] | ((uint32_t)r[5] << 16), (uint32_t)r[6] | ((uint32_t)r[7] << 16)};
    }
}

// The new tail of every sequence: the last K - 1 raw rows of [old tail | rows].  One thread per channel
// reads its column before it writes it, so the update is in place.
__global__ __launch_bounds__(256) void gdn_tail_update_kernel(const uint16_t* qkv_raw, uint32_t qkv_stride, uint16_t* tail,
                                                             GdnShape sh) {
    const uint32_t C = 2 * sh.k_heads * sh.dk + sh.v_heads * sh.dv;
    const uint32_t ch = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
    if (ch >= C) return;
    const uint32_t hist = sh.taps - 1;
    uint16_t* tl = tail + (size_t)b * hist * C;
    const uint16_t* raw = qkv_raw + (size_t)b * sh.rows * qkv_stride;
    uint16_t keep[GDN_MAX_TAPS];
#pragma unroll
    for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
        if (j >= hist) break;
        const int src = (int)sh.rows + (int)j - (int)hist;
        keep[j] = src >= 0 ? raw[(size_t)src * qkv_stride + ch] : tl[(size_t)((int)hist + src) * C + ch];
    }
#pragma unroll
    for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
        if (j >= hist) break;
        tl[(size_t)j * C + ch] = keep[j];
    }
}

// out[row, head] = rmsnorm(y) * weight * silu(z) in place over the 16-bit y rows the recurrence left in out.
template <int ACT>
__global__ __launch_bounds__(256) void gdn_gated_norm_rows_kernel(uint16_t* out, uint32_t out_stride, const uint16_t* z,
                                                                 uint32_t z_stride, const uint16_t* norm_w, GdnShape sh) {
    __shared__ float part[4];
    const uint32_t h = blockIdx.x, b = blockIdx.y;
    const uint32_t pair = threadIdx.x >> 7, i = threadIdx.x & 127u;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t t = blockIdx.z * 2u + pair;
    const bool live = t < sh.rows && i < sh.dv;
    const size_t row = (size_t)b * sh.rows + t;
    float y = 0.0f;
    if (live) y = act_to_f32<ACT>(out[row * out_stride + h * sh.dv + i]);
    const float ws = wave_sum_bcast(fmaf(y, y, 0.0f));
    if (lane == 0) part[wave] = ws;
    __syncthreads();
    if (!live) return;
    const float total = (part[2 * pair] + part[2 * pair + 1]) + (0.0f + 0.0f);
    const float inv = rsqrtf(total / (float)sh.dv + GDN_RMS_EPS);
    const float normed = y * inv * bf16_to_f32(norm_w[i]);
    const float gate = gdn_silu(act_to_f32<ACT>(z[row * z_stride + h * sh.dv + i]));
    out[row * out_stride + h * sh.dv + i] = f32_to_act<ACT>(normed * gate);
}

// The same for heads of 128 values in 16-byte pieces: sixteen lanes per (row, head), eight values per
// lane, sixteen (row, head) units per block, no barrier and no LDS.  The sum of squares is the balanced
// tree of the kernel above -- pairs, fours and eights inside the lane, then the lanes 1, 2, 4 and 8
// apart, where the kernel above goes on to its second wave -- so the result has the same bits.
// out, z and norm_w rows 16-byte aligned.
template <int ACT>
__global__ __launch_bounds__(256) void gdn_gated_norm_rows128_kernel(uint16_t* out, uint32_t out_stride, const uint16_t* z,
                                                                    uint32_t z_stride, const uint16_t* norm_w, GdnShape sh,
                                                                    uint32_t units) {
    const uint32_t u = blockIdx.x * 16u + (threadIdx.x >> 4), sub = threadIdx.x & 15u;
    const bool live = u < units;
    const uint32_t uu = live ? u : units - 1u;             // every lane takes part in the sum
    const uint32_t h = uu % sh.v_heads;
    const size_t row = uu / sh.v_heads;                    // batch * rows + t
    uint16_t* const op = out + row * out_stride + h * 128u + sub * 8u;
    const uint4 yr = *reinterpret_cast<const uint4*>(op);
    const uint4 zr = *reinterpret_cast<const uint4*>(z + row * z_stride + h * 128u + sub * 8u);
    const uint4 wr = *reinterpret_cast<const uint4*>(norm_w + sub * 8u);
    float y[8], g[8], w[8], q[8];
    act2_to_f32<ACT>(yr.x, y[0], y[1]); act2_to_f32<ACT>(yr.y, y[2], y[3]);
    act2_to_f32<ACT>(yr.z, y[4], y[5]); act2_to_f32<ACT>(yr.w, y[6], y[7]);
    act2_to_f32<ACT>(zr.x, g[0], g[1]); act2_to_f32<ACT>(zr.y, g[2], g[3]);
    act2_to_f32<ACT>(zr.z, g[4], g[5]); act2_to_f32<ACT>(zr.w, g[6], g[7]);
    act2_to_f32<ACT_BF16>(wr.x, w[0], w[1]); act2_to_f32<ACT_BF16>(wr.y, w[2], w[3]);
    act2_to_f32<ACT_BF16>(wr.z, w[4], w[5]); act2_to_f32<ACT_BF16>(wr.w, w[6], w[7]);
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = fmaf(y[j], y[j], 0.0f);
    const float lane_sum = ((q[0] + q[1]) + (q[2] + q[3])) + ((q[4] + q[5]) + (q[6] + q[7]));
    const float total = seg_reduce_sum<16>(lane_sum) + (0.0f + 0.0f);
    const float inv = rsqrtf(total / (float)sh.dv + GDN_RMS_EPS);
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = y[2 * j] * inv * w[2 * j] * gdn_silu(g[2 * j]);
        const float hi = y[2 * j + 1] * inv * w[2 * j + 1] * gdn_silu(g[2 * j + 1]);
        r[j] = (uint32_t)f32_to_act<ACT>(lo) | ((uint32_t)f32_to_act<ACT>(hi) << 16);
    }
    if (live) *reinterpret_cast<uint4*>(op) = uint4{r[0], r[1], r[2], r[3]};
}

// The recurrence alone over the rows of a call: S, and y[t] = S q rounded to 16 bits into out (the
// kernel above norms it).  A row costs a few hundred cycles of arithmetic and a trip to memory costs
// several times that, so the rows arrive a tile of 32 at a time: all 256 threads fetch the next
// tile's q, k and v rows of this head (16 bytes per load, six loads per thread at 128 x 128) into
// registers while the current tile is worked on from LDS, the threads of the first rows compute the
// tile's decays and betas, and one barrier per tile hands both over.  Inside a tile nothing waits
// for the block.  The rows of S do not depend on one another (kv, delta and y of row dv read S[dv, :]
// only), so a head's DV rows are shared out over DV / (16 GPB) blocks, each with GPB groups of sixteen
// rows: eight times as many blocks as heads at GPB = 1, and an eighth of the arithmetic per row and
// thread.  conv_out rows 16-byte aligned, DK and DV multiples of 8.
template <int ACT, int DK, int DV, bool STATE_BF16, int GPB>
__global__ __launch_bounds__(256) void gdn_delta_rows_kernel(GdnDeltaParams p) {
    constexpr int EPL = DK / 16;
    constexpr int GROUPS = DV / 16;
    constexpr uint32_t TR = 32;                             // rows per tile
    constexpr uint32_t ROW_E = 2 * DK + DV;                 // elements of a staged row: q | k | v
    constexpr uint32_t CPR = ROW_E / 8;                     // 16-byte chunks per row
    constexpr uint32_t NLD = (TR * CPR + 255) / 256;        // chunks per thread and tile
    static_assert(DK % 16 == 0 && DV % 16 == 0 && EPL >= 1 && EPL <= 16 && ROW_E % 8 == 0 && GROUPS % GPB == 0, "shape");
    const uint32_t g0 = blockIdx.z * GPB;                   // first of this block's groups of sixteen state rows
    __shared__ __attribute__((aligned(16))) uint16_t rows_s[2][TR][ROW_E];
    __shared__ float decay_s[2][TR], beta_s[2][TR];
    const uint32_t h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const uint32_t sub = tid & 15u, row_in_pass = tid >> 4;
    const GdnShape& sh = p.sh;
    const uint32_t hk = h / (sh.v_heads / sh.k_heads);
    const float exp_a = expf(bf16_to_f32(p.a_log[h]));
    const float dtb = bf16_to_f32(p.dt_bias[h]);
    const size_t state_base = (((size_t)b * sh.v_heads + h) * DV) * DK;
    float s[GPB][EPL];
#pragma unroll
    for (int g = 0; g < GPB; ++g) {
        const size_t at = state_base + (size_t)((g0 + g) * 16 + row_in_pass) * DK + sub * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e)
            s[g][e] = STATE_BF16 ? bf16_to_f32(reinterpret_cast<const uint16_t*>(p.state)[at + e])
                                 : reinterpret_cast<const float*>(p.state)[at + e];
    }
    // this thread's chunks of a tile: chunk c of the tile is row c / CPR, elements 8 (c % CPR) ..
    uint4 stage[NLD];
    uint16_t a_raw = 0, b_raw = 0;
    auto fetch_tile = [&](uint32_t t0) {
#pragma unroll
        for (uint32_t j = 0; j < NLD; ++j) {
            const uint32_t c = tid + 256 * j, r = c / CPR, e = (c % CPR) * 8;
            stage[j] = uint4{0u, 0u, 0u, 0u};
            if (c < TR * CPR && t0 + r < sh.rows) {
                const size_t row = (size_t)b * sh.rows + t0 + r;
                const uint16_t* base = p.conv_out + row * p.conv_stride;
                const uint16_t* src = e < (uint32_t)DK ? base + hk * DK + e
                                    : e < 2u * DK ? base + (sh.k_heads + hk) * DK + (e - DK)
                                                  : base + 2 * sh.k_heads * DK + h * DV + (e - 2 * DK);
                stage[j] = *reinterpret_cast<const uint4*>(src);
            }
        }
        if (tid < TR && t0 + tid < sh.rows) {
            const size_t row = (size_t)b * sh.rows + t0 + tid;
            a_raw = p.a_proj[row * p.ab_stride + h];
            b_raw = p.b_proj[row * p.ab_stride + h];
        }
    };
    auto store_tile = [&](uint32_t buf) {
#pragma unroll
        for (uint32_t j = 0; j < NLD; ++j) {
            const uint32_t c = tid + 256 * j;
            if (c < TR * CPR) *reinterpret_cast<uint4*>(&rows_s[buf][c / CPR][(c % CPR) * 8]) = stage[j];
        }
        if (tid < TR) {
            decay_s[buf][tid] = expf(-exp_a * gdn_softplus(act_to_f32<ACT>(a_raw) + dtb));
            beta_s[buf][tid] = 1.0f / (1.0f + expf(-act_to_f32<ACT>(b_raw)));
        }
    };
    fetch_tile(0);
    store_tile(0);
    __syncthreads();
    for (uint32_t t0 = 0, buf = 0; t0 < sh.rows; t0 += TR, buf ^= 1u) {
        const uint32_t n = min(TR, sh.rows - t0);
        if (t0 + TR < sh.rows) fetch_tile(t0 + TR);
        for (uint32_t u = 0; u < n; ++u) {
            const uint16_t* rs = rows_s[buf][u];
            float q[EPL], k[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) { q[e] = act_to_f32<ACT>(rs[sub * EPL + e]); k[e] = act_to_f32<ACT>(rs[DK + sub * EPL + e]); }
            const float g_decay = decay_s[buf][u], beta = beta_s[buf][u];
            uint16_t* yrow = p.out + ((size_t)b * sh.rows + t0 + u) * p.out_stride + h * DV;
#pragma unroll
            for (int g = 0; g < GPB; ++g) {
                const uint32_t dv = (g0 + g) * 16 + row_in_pass;
                float kv = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) { s[g][e] *= g_decay; kv = fmaf(s[g][e], k[e], kv); }
                kv = seg_reduce_sum<16>(kv);
                const float delta = (act_to_f32<ACT>(rs[2 * DK + dv]) - kv) * beta;
                float o = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) { s[g][e] = fmaf(k[e], delta, s[g][e]); o = fmaf(s[g][e], q[e], o); }
                o = seg_reduce_sum<16>(o);
                if (sub == 0) yrow[dv] = f32_to_act<ACT>(o);
            }
        }
        if (t0 + TR < sh.rows) store_tile(buf ^ 1u);        // the other buffer: nobody reads it during this tile
        __syncthreads();
    }
#pragma unroll
    for (int g = 0; g < GPB; ++g) {
        const size_t at = state_base + (size_t)((g0 + g) * 16 + row_in_pass) * DK + sub * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            if (STATE_BF16) reinterpret_cast<uint16_t*>(p.state)[at + e] = f32_to_bf16(s[g][e]);
            else reinterpret_cast<float*>(p.state)[at + e] = s[g][e];
        }
    }
}

// ---- one decode token: both kernels above in one launch --------------------------------------------
// Block (key head, sequence) of 256 R threads, R = Hv / Hk value heads per key head: the first 256
// threads run the conv + SiLU + norm of the key head's q and k channels (q on waves 0 - 1, k on
// waves 2 - 3: each channel on the lane it has in gdn_conv_norm_kernel, wave sums added in that
// kernel's order, so the same bits), group r of 256 threads the conv of value head Hk-head * R + r
// and then its delta rule and gated norm exactly as gdn_delta_gated_kernel does, with q, k and v
// taken from LDS instead of a conv_out row in memory.  The thread that computes a channel holds the
// channel's tail column in registers and writes it back shifted: the block is the only reader of
// its channels, so the tail is updated in place with no ordering between blocks.  The state rows
// are requested before the conv so that they arrive while it runs.
struct GdnDecodeParams {
    GdnDeltaParams d;           // conv_out unused
    const uint16_t* qkv_raw;    // [batch, qkv_stride]
    uint32_t qkv_stride;
    uint16_t* tail;             // [batch, taps - 1, C]
    const uint16_t* conv_w;     // BF16 [C, taps]
};

template <int ACT, int DK, int DV, int R, bool STATE_BF16>
__global__ __launch_bounds__(256 * R) void gdn_decode_fused_kernel(GdnDecodeParams pp) {
    constexpr int EPL = DK / 16;
    constexpr int GROUPS = DV / 16;
    static_assert(DK <= 128 && DV <= 256 /* one channel per thread */ && DK % 16 == 0 && DV % 16 == 0, "shape");
    __shared__ float q_s[DK], k_s[DK];
    __shared__ float v_s[R][DV], y_s[R][DV];
    __shared__ float part_qk[4], part[R][4];
    const GdnDeltaParams& p = pp.d;
    const GdnShape& sh = p.sh;
    const uint32_t hk = blockIdx.x, b = blockIdx.y;
    const uint32_t r = threadIdx.x >> 8, lt = threadIdx.x & 255u;          // value head of the group, thread in the group
    const uint32_t lane = lt & 63u, wave = lt >> 6;
    const uint32_t h = hk * R + r;
    const uint32_t sub = lt & 15u, row_in_pass = lt >> 4;
    const uint32_t C = 2 * sh.k_heads * DK + sh.v_heads * DV;
    const uint32_t hist = sh.taps - 1;

    // ---- the state rows of this value head
    const size_t state_base = (((size_t)b * sh.v_heads + h) * DV) * DK;
    float s[GROUPS][EPL];
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const size_t at = state_base + (size_t)(g * 16 + row_in_pass) * DK + sub * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e)
            s[g][e] = STATE_BF16 ? bf16_to_f32(reinterpret_cast<const uint16_t*>(p.state)[at + e])
                                 : reinterpret_cast<const float*>(p.state)[at + e];
    }

    // everything else the token needs from memory is requested now as well, ahead of the conv's barriers
    const size_t row = b;
    const uint16_t a_raw = p.a_proj[row * p.ab_stride + h], b_raw = p.b_proj[row * p.ab_stride + h];
    const uint16_t a_log_raw = p.a_log[h], dt_raw = p.dt_bias[h];
    const uint16_t z_raw = lt < (uint32_t)DV ? p.z[row * p.z_stride + h * DV + lt] : (uint16_t)0;
    const uint16_t nw_raw = lt < (uint32_t)DV ? p.norm_w[lt] : (uint16_t)0;

    // ---- conv + SiLU of one channel, tail column shifted in place; returns the 16-bit result as a float
    uint16_t* tl = pp.tail + (size_t)b * hist * C;
    const uint16_t* raw = pp.qkv_raw + (size_t)b * pp.qkv_stride;
    auto conv_channel = [&](uint32_t ch) -> float {
        uint16_t x[GDN_MAX_TAPS];
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            if (j > hist) break;
            x[j] = j < hist ? tl[(size_t)j * C + ch] : raw[ch];
        }
        float acc = 0.0f;
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            if (j > hist) break;
            acc = fmaf(act_to_f32<ACT>(x[j]), bf16_to_f32(pp.conv_w[ch * sh.taps + j]), acc);
        }
#pragma unroll
        for (uint32_t j = 0; j < GDN_MAX_TAPS; ++j) {
            if (j >= hist) break;
            tl[(size_t)j * C + ch] = x[j + 1];
        }
        return act_to_f32<ACT>(f32_to_act<ACT>(gdn_silu(acc)));
    };
    // q: threads 0 .. DK - 1 of group 0; k: threads 128 .. 128 + DK - 1 of group 0
    const bool is_q = r == 0 && lt < (uint32_t)DK, is_k = r == 0 && lt >= 128u && lt < 128u + (uint32_t)DK;
    float qk = 0.0f;
    if (is_q) qk = conv_channel(hk * DK + lt);
    if (is_k) qk = conv_channel(sh.k_heads * DK + hk * DK + (lt - 128u));
    if (lt < (uint32_t)DV) v_s[r][lt] = conv_channel(2 * sh.k_heads * DK + h * DV + lt);
    if (r == 0) {
        const float ws = wave_sum_bcast(qk * qk);               // fma(x, x, 0) of the separate kernel
        if (lane == 0) part_qk[wave] = ws;
    }
    __syncthreads();
    if (is_q || is_k) {
        const float total = is_q ? (part_qk[0] + part_qk[1]) + (0.0f + 0.0f) : (part_qk[2] + part_qk[3]) + (0.0f + 0.0f);
        // the divisor and the k scale from the run-time shape, as gdn_conv_norm_kernel takes them
        const float inv = rsqrtf(total / (float)sh.dk + GDN_RMS_EPS);
        const float scale = is_q ? 1.0f / (float)sh.dk : rsqrtf((float)sh.dk);
        const float o = act_to_f32<ACT>(f32_to_act<ACT>(qk * inv * scale));
        if (is_q) q_s[lt] = o; else k_s[lt - 128u] = o;
    }
    __syncthreads();

    // ---- delta rule + gated norm of value head h (gdn_delta_gated_kernel, one row)
    const float exp_a = expf(bf16_to_f32(a_log_raw));
    const float dtb = bf16_to_f32(dt_raw);
    float q[EPL], k[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) { q[e] = q_s[sub * EPL + e]; k[e] = k_s[sub * EPL + e]; }
    const float g_decay = expf(-exp_a * gdn_softplus(act_to_f32<ACT>(a_raw) + dtb));
    const float beta = 1.0f / (1.0f + expf(-act_to_f32<ACT>(b_raw)));
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const uint32_t dv = g * 16 + row_in_pass;
        float kv = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) { s[g][e] *= g_decay; kv = fmaf(s[g][e], k[e], kv); }
        kv = seg_reduce_sum<16>(kv);
        const float delta = (v_s[r][dv] - kv) * beta;
        float o = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) { s[g][e] = fmaf(k[e], delta, s[g][e]); o = fmaf(s[g][e], q[e], o); }
        o = seg_reduce_sum<16>(o);
        if (sub == 0) y_s[r][dv] = act_to_f32<ACT>(f32_to_act<ACT>(o));
    }
    __syncthreads();
    float sumsq = 0.0f;
    if (lt < (uint32_t)DV) sumsq = fmaf(y_s[r][lt], y_s[r][lt], sumsq);
    sumsq = wave_sum_bcast(sumsq);
    if (lane == 0) part[r][wave] = sumsq;
    __syncthreads();
    const float total = (part[r][0] + part[r][1]) + (part[r][2] + part[r][3]);
    const float inv = rsqrtf(total / (float)DV + GDN_RMS_EPS);
    if (lt < (uint32_t)DV) {
        const float normed = y_s[r][lt] * inv * bf16_to_f32(nw_raw);
        const float gate = gdn_silu(act_to_f32<ACT>(z_raw));
        p.out[row * p.out_stride + h * DV + lt] = f32_to_act<ACT>(normed * gate);
    }
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const size_t at = state_base + (size_t)(g * 16 + row_in_pass) * DK + sub * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            if (STATE_BF16) reinterpret_cast<uint16_t*>(p.state)[at + e] = f32_to_bf16(s[g][e]);
            else reinterpret_cast<float*>(p.state)[at + e] = s[g][e];
        }
    }
}

}  // namespace nvmai
