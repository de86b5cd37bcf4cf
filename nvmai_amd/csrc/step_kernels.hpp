// The small operators around the MoE block of a decode step: RMSNorm, affine embedding lookup,
// and the fused greedy LM head (RMSNorm -> one logit per vocabulary row -> argmax).  gfx950.
#pragma once

#include "common.hpp"

namespace nvmai {

// ---- RMSNorm -------------------------------------------------------------------------
// y = x * inv * w, inv = 1 / sqrt(mean(x^2) + eps) (rmsnorm.metal:31-62, 83-87); no weight:
// y = x * inv (:152-175).  A row may be one head of a [heads, head_dim] vector (:101-148).
// One wave per row.  The sum of squares has a fixed order so that a CPU run of the same order
// gives the same bits: lane l runs acc = fma(x, x, acc) over the elements l, l + 64, ...,
// then an xor butterfly 32, 16, 8, 4, 2, 1; every later step is one IEEE operation.
// (rms_wave_sum and rms_inverse, the stated order and the single IEEE steps, are in common.hpp)

// One wave per row.  STAGED: the row travels through LDS -- 16-byte loads in, the per-lane sums
// and products read and written two bytes at a time there, 16-byte stores out -- so that a lane's
// 32 strided elements of a 2048-wide row are not 32 dependent trips to memory (23 us per row that
// way, a few us staged); the arithmetic and its order are the same either way.  delta != nullptr:
// the row is first replaced by round(row + delta) (the residual add, utility.metal:95-104) and
// stored back.  Rows need 16-byte alignment and d a multiple of 8 for the staged form (the entry
// point checks); lds holds 4 rows of d elements.
// DFIX: the row length when it is known at compile time (the loops then unroll and a lane's
// LDS reads are all in flight together), 0 = any.
template <int ACT, bool STAGED, int DFIX>
__device__ __forceinline__ void rms_row(uint16_t* xr, const uint16_t* dr, const uint16_t* weight, uint16_t* o,
                                        uint32_t d_any, float eps, uint16_t* row_s, uint32_t lane) {
    const uint32_t d = DFIX ? (uint32_t)DFIX : d_any;
    if (STAGED) {
        for (uint32_t c = lane; c < d / 8; c += 64) {
            uint4 v = *reinterpret_cast<const uint4*>(xr + c * 8);
            if (dr) {
                const uint4 dl = *reinterpret_cast<const uint4*>(dr + c * 8);
                uint32_t* vv = reinterpret_cast<uint32_t*>(&v);
                const uint32_t* dd = reinterpret_cast<const uint32_t*>(&dl);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float a0, a1, b0, b1;
                    act2_to_f32<ACT>(vv[j], a0, a1);
                    act2_to_f32<ACT>(dd[j], b0, b1);
                    vv[j] = (uint32_t)f32_to_act<ACT>(__fadd_rn(a0, b0)) | ((uint32_t)f32_to_act<ACT>(__fadd_rn(a1, b1)) << 16);
                }
                *reinterpret_cast<uint4*>(xr + c * 8) = v;
            }
            *reinterpret_cast<uint4*>(row_s + c * 8) = v;
        }
        __builtin_amdgcn_wave_barrier();
    } else if (dr) {
        for (uint32_t i = lane; i < d; i += 64)
            xr[i] = f32_to_act<ACT>(__fadd_rn(act_to_f32<ACT>(xr[i]), act_to_f32<ACT>(dr[i])));
    }
    const uint16_t* src = STAGED ? row_s : xr;
    float acc = 0.0f;
#pragma unroll
    for (uint32_t i = lane; i < d; i += 64) {
        const float v = act_to_f32<ACT>(src[i]);
        acc = fmaf(v, v, acc);
    }
    const float inv = rms_inverse(rms_wave_sum(acc), d, eps);
    uint16_t* dst = STAGED ? row_s : o;
#pragma unroll
    for (uint32_t i = lane; i < d; i += 64) {       // in place is fine: a lane rereads only what it writes
        float v = __fmul_rn(act_to_f32<ACT>(src[i]), inv);
        if (weight) v = __fmul_rn(v, bf16_to_f32(weight[i]));
        dst[i] = f32_to_act<ACT>(v);
    }
    if (STAGED) {
        __builtin_amdgcn_wave_barrier();
        for (uint32_t c = lane; c < d / 8; c += 64)
            *reinterpret_cast<uint4*>(o + c * 8) = *reinterpret_cast<const uint4*>(row_s + c * 8);
    }
}

// weight_s: the block's copy of the norm weight in LDS (staged form), read two bytes at a time
template <int ACT, bool STAGED, int DFIX>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* x, uint32_t x_stride, const uint16_t* weight,
                                                      uint16_t* out, uint32_t out_stride, uint32_t rows, uint32_t d,
                                                      float eps) {
    extern __shared__ __attribute__((aligned(16))) uint16_t rms_lds[];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint16_t* w = weight;
    if (STAGED && weight) {
        for (uint32_t c = threadIdx.x; c < d / 8; c += 256)
            *reinterpret_cast<uint4*>(rms_lds + 4 * d + c * 8) = *reinterpret_cast<const uint4*>(weight + c * 8);
        __syncthreads();
        w = rms_lds + 4 * d;
    }
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= rows) return;                       // uniform per wave, after the block's only barrier
    // out may be x: the row is complete in LDS (or every lane rereads only its own elements) before it is written
    rms_row<ACT, STAGED, DFIX>(const_cast<uint16_t*>(x) + (size_t)row * x_stride, nullptr, w, out + (size_t)row * out_stride,
                         d, eps, rms_lds + wave * d, lane);
}

// hidden += delta (rounded to the activation type and stored, utility.metal:95-104), then
// out = RMSNorm(hidden) * weight of the updated row (rmsnorm.metal:64-110): the residual add that
// ends one block of a layer and the norm that opens the next, in one pass over the row.  Same
// arithmetic and summation order as the two kernels one after the other.
template <int ACT, bool STAGED, int DFIX>
__global__ __launch_bounds__(256) void residual_add_rmsnorm_kernel(uint16_t* hidden, uint32_t hidden_stride,
                                                                   const uint16_t* delta, uint32_t delta_stride,
                                                                   const uint16_t* weight, uint16_t* out,
                                                                   uint32_t out_stride, uint32_t rows, uint32_t d,
                                                                   float eps) {
    extern __shared__ __attribute__((aligned(16))) uint16_t rms_lds[];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint16_t* w = weight;
    if (STAGED && weight) {
        for (uint32_t c = threadIdx.x; c < d / 8; c += 256)
            *reinterpret_cast<uint4*>(rms_lds + 4 * d + c * 8) = *reinterpret_cast<const uint4*>(weight + c * 8);
        __syncthreads();
        w = rms_lds + 4 * d;
    }
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= rows) return;                       // uniform per wave, after the block's only barrier
    rms_row<ACT, STAGED, DFIX>(hidden + (size_t)row * hidden_stride, delta + (size_t)row * delta_stride, w,
                         out + (size_t)row * out_stride, d, eps, rms_lds + wave * d, lane);
}

// A few rows of a width known at compile time (a decode step's hidden rows): one wave per block and
// row, no LDS.  Lane l loads its elements l, l + 64, ... with two-byte loads -- the 64 lanes of one
// instruction read 128 contiguous bytes, and with the width fixed all of a lane's loads (row,
// delta, weight) are in flight together, so the kernel is one trip to memory, the fma chain, the
// butterfly and the stores.  Same arithmetic and order as rms_row.
template <int ACT, int DFIX, bool RESIDUAL>
__global__ __launch_bounds__(64) void rms_direct_kernel(uint16_t* x, uint32_t x_stride, const uint16_t* delta,
                                                        uint32_t delta_stride, const uint16_t* weight, uint16_t* out,
                                                        uint32_t out_stride, float eps) {
    constexpr int N = DFIX / 64;
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    uint16_t* xr = x + (size_t)row * x_stride;
    const uint16_t* dr = RESIDUAL ? delta + (size_t)row * delta_stride : nullptr;
    uint16_t* o = out + (size_t)row * out_stride;
    uint16_t xv[N], dv[N], wv[N];
#pragma unroll
    for (int j = 0; j < N; ++j) xv[j] = xr[lane + 64 * j];
    if (RESIDUAL) {
#pragma unroll
        for (int j = 0; j < N; ++j) dv[j] = dr[lane + 64 * j];
    }
    if (weight) {
#pragma unroll
        for (int j = 0; j < N; ++j) wv[j] = weight[lane + 64 * j];
    }
    float v[N];
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < N; ++j) {
        if (RESIDUAL) {
            xv[j] = f32_to_act<ACT>(__fadd_rn(act_to_f32<ACT>(xv[j]), act_to_f32<ACT>(dv[j])));
            xr[lane + 64 * j] = xv[j];
        }
        v[j] = act_to_f32<ACT>(xv[j]);
        acc = fmaf(v[j], v[j], acc);
    }
    const float inv = rms_inverse(rms_wave_sum(acc), DFIX, eps);
#pragma unroll
    for (int j = 0; j < N; ++j) {
        float y = __fmul_rn(v[j], inv);
        if (weight) y = __fmul_rn(y, bf16_to_f32(wv[j]));
        o[lane + 64 * j] = f32_to_act<ACT>(y);
    }
}

// ---- epilogue of the fused q / k / v projection of a full-attention layer --------------------------
// One wave per head of one token, replacing split_q_gate + rmsnorm_bf16w_perhead (q, k) + rope_neox_subdim
// (q, k) (RealForwardRunner.swift:2213-2255; the reference's own fusion of the norm and the rotation is
// fused_qkv_epilogue, fused.metal:72-162):
//   q head h:  packed [q ; gate] -> gate copied out, q = rope(round(rmsnorm(q) * q_weight))
//   k head h:  k = rope(round(rmsnorm(k) * k_weight)) into the K stage row
//   v head h:  copied into the V stage row (v_norm: RMS norm without weight first, as the
//              reference's fused kernel has it for models that norm V)
// The norm is the arithmetic of rmsnorm_kernel (same summation order), the result is rounded to the
// activation type before the rotation as the separate kernels hand it over, and the rotation is the
// arithmetic of rope_neox_subdim_kernel: the outputs are the same bits as the five launches.
struct QkvEpilogueParams {
    const uint16_t* proj;       // [tokens, proj_stride]: q heads packed [q ; gate], then k heads, then v heads
    uint32_t proj_stride;
    uint32_t q_packed;          // 1: q heads are [q ; gate] pairs (2 head_dim each); 0: plain q heads, no gate
    const uint16_t* q_weight;   // BF16 [head_dim] or NULL
    const uint16_t* k_weight;
    uint16_t* q_out;            // [tokens, num_q_heads, head_dim]
    uint16_t* gate_out;         // [tokens, num_q_heads, head_dim] (q_packed only)
    uint16_t* k_out;            // [tokens, kv_stride]
    uint16_t* v_out;
    uint32_t kv_stride;
    uint32_t tokens, num_q_heads, num_kv_heads, head_dim, rotary_dim;
    uint32_t v_norm;
    const uint32_t* positions;  // one per token, or NULL = position0
    uint32_t position0;
    float theta, eps;
    // Optional quantize-on-write of the finished k / v heads (KVCacheQuantizer.encode,
    // kv_cache_quantize.metal:7-73), head_dim a multiple of 64: token t's row at
    // kc / vc + t * kv_row_stride bytes = [codes | fp16 scales | fp16 biases] of kv_bits bits.  A wave
    // holds one group of 64 elements per pass of its store loop, so the group's extremes are two
    // butterflies over the lanes: the arithmetic, and so the bits, of kv_quantize_kernel.
    uint8_t* kc;
    uint8_t* vc;
    uint32_t kv_bits, kv_row_stride, kv_value_bytes;
};

template <int ACT, int HD>
__global__ __launch_bounds__(256) void qkv_epilogue_kernel(QkvEpilogueParams p) {
    // HD: the head size when it is known at compile time (0 = any, read from p): the loops over a
    // head's elements then unroll, and a lane's loads of a pass are in flight together
    __shared__ uint16_t head_s[4][512];
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t heads = p.num_q_heads + 2 * p.num_kv_heads;
    const uint32_t hidx = blockIdx.x * 4 + wave, token = blockIdx.y;
    if (hidx >= heads) return;                              // wave-uniform; no block-wide barrier below
    const uint32_t hd = HD ? (uint32_t)HD : p.head_dim;
    const bool is_q = hidx < p.num_q_heads, is_k = !is_q && hidx < p.num_q_heads + p.num_kv_heads;
    const uint32_t q_span = p.q_packed ? 2 * hd : hd;
    const uint16_t* src;
    uint16_t* dst;
    const uint16_t* w = nullptr;
    uint8_t* cache = nullptr;                                // this token's cache row (k / v heads of a fused call)
    uint32_t kv_elem0 = 0;                                  // first element of this head in the row
    if (is_q) {
        src = p.proj + (size_t)token * p.proj_stride + hidx * q_span;
        dst = p.q_out + ((size_t)token * p.num_q_heads + hidx) * hd;
        w = p.q_weight;
        if (p.q_packed) {
            uint16_t* g = p.gate_out + ((size_t)token * p.num_q_heads + hidx) * hd;
#pragma unroll
            for (uint32_t i = lane; i < hd; i += 64) g[i] = src[hd + i];
        }
    } else {
        const uint32_t kvh = hidx - p.num_q_heads - (is_k ? 0 : p.num_kv_heads);
        src = p.proj + (size_t)token * p.proj_stride + p.num_q_heads * q_span + (is_k ? 0 : p.num_kv_heads * hd) + kvh * hd;
        uint16_t* stage = is_k ? p.k_out : p.v_out;
        dst = stage ? stage + (size_t)token * p.kv_stride + kvh * hd : nullptr;
        w = is_k ? p.k_weight : nullptr;
        uint8_t* cbase = is_k ? p.kc : p.vc;
        if (cbase) cache = cbase + (size_t)token * p.kv_row_stride;
        kv_elem0 = kvh * hd;
    }
    uint16_t* hs = head_s[wave];
    const bool norm = is_q || is_k || p.v_norm;
    if (norm) {
        float acc = 0.0f;
#pragma unroll
        for (uint32_t i = lane; i < hd; i += 64) {
            const float v = act_to_f32<ACT>(src[i]);
            acc = fmaf(v, v, acc);
        }
        const float inv = rms_inverse(rms_wave_sum(acc), hd, p.eps);
#pragma unroll
        for (uint32_t i = lane; i < hd; i += 64) {
            float v = __fmul_rn(act_to_f32<ACT>(src[i]), inv);
            if (w) v = __fmul_rn(v, bf16_to_f32(w[i]));
            hs[i] = f32_to_act<ACT>(v);
        }
    } else {
#pragma unroll
        for (uint32_t i = lane; i < hd; i += 64) hs[i] = src[i];
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xC07F);                      // lgkmcnt(0): this wave's LDS writes have landed
    const uint32_t half_rot = (is_q || is_k) ? p.rotary_dim / 2 : 0;
    const uint32_t pos = p.positions ? p.positions[token] : p.position0;
#pragma unroll
    for (uint32_t i = lane; i < hd; i += 64) {
        uint16_t o = hs[i];
        if (i < 2 * half_rot) {
            const uint32_t pair = i < half_rot ? i : i - half_rot;
            const float exponent = __fdiv_rn(-(float)(2u * pair), (float)p.rotary_dim);
            const float angle = __fmul_rn((float)pos, powf(p.theta, exponent));
            const float c = cosf(angle), s = sinf(angle);
            const float x0 = act_to_f32<ACT>(hs[pair]), x1 = act_to_f32<ACT>(hs[half_rot + pair]);
            o = i < half_rot ? f32_to_act<ACT>(__fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s)))
                             : f32_to_act<ACT>(__fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c)));
        }
        if (dst) dst[i] = o;
        if (cache) {                                        // wave-uniform; hd % 64 == 0: every lane holds an element
            const float v = act_to_f32<ACT>(o);
            float mn = v, mx = v;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                mn = fminf(mn, shfl_xor_f(mn, off));
                mx = fmaxf(mx, shfl_xor_f(mx, off));
            }
            const float levels = p.kv_bits == 4 ? 15.0f : 255.0f;
            const float bias = mn;
            const float scale = mx > mn ? __fdiv_rn(__fsub_rn(mx, mn), levels) : 0.0f;
            const uint32_t groups = p.num_kv_heads * hd / 64, g = (kv_elem0 + i) / 64, e = kv_elem0 + i;
            if (lane == 0) {
                reinterpret_cast<uint16_t*>(cache + p.kv_value_bytes)[g] = f32_to_f16(scale);
                reinterpret_cast<uint16_t*>(cache + p.kv_value_bytes)[groups + g] = f32_to_f16(bias);
            }
            float q = 0.0f;
            if (scale > 0.0f) q = roundf(fminf(fmaxf(__fdiv_rn(__fsub_rn(v, bias), scale), 0.0f), levels));
            const uint32_t code = (uint32_t)q;
            if (p.kv_bits == 8) {
                cache[e] = (uint8_t)code;
            } else {
                const uint32_t hi = shfl_xor_u(code, 1);
                if ((lane & 1) == 0) cache[e / 2] = (uint8_t)(code | (hi << 4));
            }
        }
    }
}

// ---- dense BF16 rows against a few BF16 inputs (the BF16 LM head) ---------------------------------
// y[t, r] = sum_k W[r, k] x[t, k] for up to 16 inputs per pass, on the matrix cores: the weight rows
// are the B operand of v_mfma_f32_16x16x32_bf16 exactly as they lie in memory -- lane (i = lane % 16,
// q = lane / 16) loads the 32 bytes W[r0 + i, k0 + 16 q .. + 16), so four lanes cover 128 contiguous
// bytes of a row and every byte of the matrix is read once -- and the inputs are the A operand,
// staged once per block in LDS (rows 16 bytes apart from a power of two, so the sixteen inputs of a
// fragment read fall into different banks).  Only the inputs that exist are staged: row t of A
// reaches row t of the product alone, and the rows of absent inputs are never stored, so their lanes
// read the last staged input again -- at one input a block holds 4 KB of LDS instead of 64 and the
// resident waves per CU are bounded by registers.  A wave owns 16 rows at a time and keeps DEPTH
// super-steps of 64 k in flight.  The product is bound by the matrix's bytes: the matrix cores
// idle most of the time, which is what lets one kernel serve 1 to 16 inputs at the same speed.
typedef __bf16 dg_bf8_t __attribute__((ext_vector_type(8)));
typedef float dg_fl4_t __attribute__((ext_vector_type(4)));
constexpr int DENSE_TOK = 16;
constexpr int DENSE_DEPTH = 4;

__global__ __launch_bounds__(256) void dense_bf16_gemv_kernel(const uint16_t* w, const uint16_t* x, uint32_t x_stride,
                                                             uint32_t tokens, uint32_t m, uint32_t n, uint16_t* y,
                                                             float* y_f32, uint32_t y_stride, uint32_t row_groups_per_block) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dense_lds[];
    const uint32_t ld = n * 2u + 16u;                       // bytes between two inputs in LDS
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t li = lane & 15u, lq = lane >> 4;
    // inputs -> LDS
    for (uint32_t c = tid; c < tokens * (n / 8u); c += 256u) {
        const uint32_t t = c / (n / 8u), k8 = c % (n / 8u);
        *reinterpret_cast<uint4*>(dense_lds + t * ld + k8 * 16u) =
            *reinterpret_cast<const uint4*>(x + (size_t)t * x_stride + k8 * 8u);
    }
    __syncthreads();
    const uint32_t steps = n / 64u;                         // super-steps of 64 k: two MFMAs each
    const uint8_t* xa = dense_lds + min(li, tokens - 1u) * ld + lq * 32u;   // this lane's A fragments
    for (uint32_t g = 0; g < row_groups_per_block; ++g) {
        const uint32_t r0 = ((blockIdx.x * row_groups_per_block + g) * 4u + wave) * 16u;
        if (r0 >= m) break;                                 // wave-uniform
        const uint32_t r = min(r0 + li, m - 1u);            // rows past the end repeat the last one, never stored
        const uint4* wp = reinterpret_cast<const uint4*>(w + (size_t)r * n + lq * 16u);
        dg_fl4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        uint4 buf[DENSE_DEPTH][2];
#pragma unroll
        for (int d = 0; d < DENSE_DEPTH; ++d) {
            const uint32_t st = min((uint32_t)d, steps - 1u);
            buf[d][0] = wp[st * 8u];
            buf[d][1] = wp[st * 8u + 1u];
        }
        for (uint32_t s0 = 0; s0 < steps; s0 += DENSE_DEPTH) {
#pragma unroll
            for (int d = 0; d < DENSE_DEPTH; ++d) {
                const uint32_t st = s0 + d;
                const uint4 b0 = buf[d][0], b1 = buf[d][1];
                const uint32_t nx = min(st + DENSE_DEPTH, steps - 1u);     // unconditional: past the end rereads the last step
                buf[d][0] = wp[nx * 8u];
                buf[d][1] = wp[nx * 8u + 1u];
                if (st < steps) {                           // uniform
                    const uint4 a0 = *reinterpret_cast<const uint4*>(xa + st * 128u);
                    const uint4 a1 = *reinterpret_cast<const uint4*>(xa + st * 128u + 16u);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dg_bf8_t, a0), __builtin_bit_cast(dg_bf8_t, b0), acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dg_bf8_t, a1), __builtin_bit_cast(dg_bf8_t, b1), acc, 0, 0, 0);
                }
            }
        }
        // acc[j] = y[input 4 q + j, row r0 + i]
        if (r0 + li < m) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t t = lq * 4u + j;
                if (t < tokens) {
                    if (y) y[(size_t)t * y_stride + r0 + li] = f32_to_bf16(acc[j]);
                    if (y_f32) y_f32[(size_t)t * y_stride + r0 + li] = acc[j];
                }
            }
        }
    }
}

// ---- elementwise helpers of the layer loop (utility.metal) -----------------------------------
// 16-bit activations in and out, fp32 arithmetic, one rounding at the end.
enum ElementwiseOp : int {
    EW_SILU_MUL = 0,        // out = silu(a) * b, silu(g) = g / (1 + exp(-g))   utility.metal:32-45
    EW_SIGMOID_MUL = 1,     // out = a / (1 + exp(-b[i]))                        :47-58
    EW_SIGMOID_SCALAR = 2,  // out = a / (1 + exp(-b[0]))                        :60-72
    EW_ADD = 3              // out = a + b                                       :95-104
};

template <int ACT, int OP>
__global__ __launch_bounds__(256) void elementwise_kernel(const uint16_t* a, const uint16_t* b, uint16_t* out,
                                                          uint32_t count) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const float x = act_to_f32<ACT>(a[i]);
    const float y = act_to_f32<ACT>(b[OP == EW_SIGMOID_SCALAR ? 0 : i]);
    float r;
    if (OP == EW_SILU_MUL) r = __fmul_rn(__fdiv_rn(x, __fadd_rn(1.0f, expf(-x))), y);
    else if (OP == EW_ADD) r = __fadd_rn(x, y);
    else r = __fdiv_rn(x, __fadd_rn(1.0f, expf(-y)));
    out[i] = f32_to_act<ACT>(r);
}

// The same, eight values (16 bytes) per thread: a, b and out 16-byte aligned, count a multiple of 8.
template <int ACT, int OP>
__global__ __launch_bounds__(256) void elementwise8_kernel(const uint16_t* a, const uint16_t* b, uint16_t* out,
                                                           uint32_t count8) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count8) return;
    const uint4 av = reinterpret_cast<const uint4*>(a)[i];
    uint4 bv = uint4{0, 0, 0, 0};
    if (OP != EW_SIGMOID_SCALAR) bv = reinterpret_cast<const uint4*>(b)[i];
    const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
    float scalar = 0.0f;
    if (OP == EW_SIGMOID_SCALAR) scalar = act_to_f32<ACT>(b[0]);
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float x[2], y[2], o[2];
        act2_to_f32<ACT>(aw[j], x[0], x[1]);
        act2_to_f32<ACT>(bw[j], y[0], y[1]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (OP == EW_SILU_MUL) o[h] = __fmul_rn(__fdiv_rn(x[h], __fadd_rn(1.0f, expf(-x[h]))), y[h]);
            else if (OP == EW_ADD) o[h] = __fadd_rn(x[h], y[h]);
            else if (OP == EW_SIGMOID_SCALAR) o[h] = __fdiv_rn(x[h], __fadd_rn(1.0f, expf(-scalar)));
            else o[h] = __fdiv_rn(x[h], __fadd_rn(1.0f, expf(-y[h])));
        }
        r[j] = (uint32_t)f32_to_act<ACT>(o[0]) | ((uint32_t)f32_to_act<ACT>(o[1]) << 16);
    }
    reinterpret_cast<uint4*>(out)[i] = uint4{r[0], r[1], r[2], r[3]};
}

// split (JOIN = false): packed [rows, 2 dim] -> lo [rows, dim], hi [rows, dim]   (split_q_gate_fp16, :75-92)
// join  (JOIN = true):  lo, hi [rows, dim]   -> packed [rows, 2 dim]             (concat_rows_fp16, :107-121)
template <bool JOIN>
__global__ __launch_bounds__(256) void split_join_rows_kernel(uint16_t* packed, uint16_t* lo, uint16_t* hi,
                                                              uint32_t rows, uint32_t dim) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * dim) return;
    const uint32_t r = i / dim, c = i % dim;
    if (JOIN) {
        packed[(size_t)r * 2 * dim + c] = lo[i];
        packed[(size_t)r * 2 * dim + dim + c] = hi[i];
    } else {
        lo[i] = packed[(size_t)r * 2 * dim + c];
        hi[i] = packed[(size_t)r * 2 * dim + dim + c];
    }
}

// ---- embedding lookup ------------------------------------------------------------------
// out[t, i] = ((float(q) * s + b) * out_scale) for row token[t] of a 4- or 8-bit affine table,
// zeros for a token id at or past vocab (dequant_int4.metal:63-91; a block of tokens:
// prefill.metal:59).  One thread per eight elements.
template <int ACT>
__global__ __launch_bounds__(256) void embed_lookup_kernel(const uint8_t* table, const uint16_t* scales,
                                                           const uint16_t* biases, uint32_t bits,
                                                           const uint32_t* token_ids, uint32_t token_id,
                                                           uint16_t* out, uint32_t out_stride, uint32_t d,
                                                           uint32_t vocab, float out_scale) {
    const uint32_t t = blockIdx.y;
    const uint32_t e0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (e0 >= d) return;
    const uint32_t tok = token_ids ? token_ids[t] : token_id;
    uint16_t* o = out + (size_t)t * out_stride + e0;
    const uint32_t n = min(8u, d - e0);
    if (tok >= vocab) {
        for (uint32_t j = 0; j < n; ++j) o[j] = 0;
        return;
    }
    const uint32_t groups = d / NVMAI_GROUP;
    const uint8_t* row = table + (size_t)tok * ((size_t)d * bits / 8);
    const float s = bf16_to_f32(scales[(size_t)tok * groups + e0 / NVMAI_GROUP]);
    const float b = bf16_to_f32(biases[(size_t)tok * groups + e0 / NVMAI_GROUP]);
    for (uint32_t j = 0; j < n; ++j) {
        const uint32_t e = e0 + j;
        const uint32_t q = bits == 8 ? row[e] : ((row[e >> 1] >> ((e & 1u) * 4u)) & 0xFu);
        o[j] = f32_to_act<ACT>(__fmul_rn(__fadd_rn(__fmul_rn((float)q, s), b), out_scale));
    }
}

// ---- greedy LM head ------------------------------------------------------------------------
// LMHeadChainInt4.encodeGreedyDecode (LMHeadChainInt4.swift:58-130; kernels logit.metal:761-937):
// token = argmax over the vocabulary rows of W[row] . norm(hidden), finite logits only, ties to
// the lower index, 0 when no logit is finite.  The RMSNorm is done inside every block (the row
// is a few KB) and rounded to the activation type as the reference stores it.
//
// One half-wave (32 lanes) per vocabulary row, in the same fixed order as the router logits so
// that the token can be compared with a CPU run of that order: lane l owns the 16-byte chunks
// l, l + 32, ... of the row; in a chunk dot = fma(q, x, dot) and xs = xs + x run in element
// order, then acc = fma(s, dot, acc), acc = fma(b, xs, acc); xor butterfly 16, 8, 4, 2, 1.
// A lane's inputs and their chunk sums do not depend on the row: they are fetched once per block
// into registers, and the block walks LMH_ROWS rows, the next row's codes in flight while the
// current one is summed.  Each block leaves (best logit, index) and a second small launch picks
// the winner.
constexpr uint32_t LMH_ROWS = 128;                // rows per block: 16 per half-wave
constexpr int LMH_STEPS = LMH_ROWS / 8;
constexpr int LMH_BUFS = 2;                       // register buffers of codes: LMH_BUFS - 1 rows in flight per half-wave

struct LmHeadParams {
    const uint16_t* hidden;       // [tokens, hidden_stride] activations
    uint32_t hidden_stride;
    const uint16_t* norm_weight;  // optional bf16 [d]
    const uint8_t* weights;       // [vocab, d * bits / 8]
    const uint16_t* scales;       // bf16 [vocab, d / 64]
    const uint16_t* biases;
    uint32_t d, vocab;
    float eps;
    float2* summaries;            // [tokens, gridDim.x] (best logit, index bits)
};

// (at least three blocks per CU where a lane holds 64 inputs: left alone, the scheduler hoists
// every load of the unrolled loop and takes all 256 registers, which leaves two waves per SIMD to
// hide each row's butterfly; with 128 inputs per lane three blocks would spill)
template <int ACT, int BITS, int CPL>
__global__ __launch_bounds__(256, (CPL * (128 / BITS) > 64 ? 2 : 3)) void lm_head_greedy_kernel(LmHeadParams p) {
    constexpr int EPC = Chunk<BITS>::elems;
    // LDS: [d] normed inputs as floats | 16 words of block results | [d] hidden row, [d] norm weight (16 bit)
    extern __shared__ float lmh_lds[];
    float* xn = lmh_lds;
    uint16_t* hraw = reinterpret_cast<uint16_t*>(lmh_lds + p.d + 16);
    uint16_t* wraw = hraw + p.d;
    const uint32_t t = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const uint16_t* h = p.hidden + (size_t)t * p.hidden_stride;

    const uint32_t hw = tid >> 5, hl = tid & 31;
    const uint32_t chunks = p.d * BITS / 128, groups = p.d / NVMAI_GROUP, row_bytes = p.d * BITS / 8;
    const uint32_t row0 = blockIdx.x * LMH_ROWS;
    const uint32_t row_end = min(row0 + LMH_ROWS, p.vocab);
    uint4 q[LMH_BUFS][CPL];
    uint16_t sc[LMH_BUFS][CPL], bi[LMH_BUFS][CPL];
    auto load_row = [&](int buf, uint32_t row) {
        row = min(row, p.vocab - 1);
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const uint32_t chunk = min(hl + 32 * c, chunks - 1);    // a lane without a chunk loads the last one
            q[buf][c] = *reinterpret_cast<const uint4*>(p.weights + (size_t)row * row_bytes + chunk * 16);
            const uint32_t g = chunk * EPC / NVMAI_GROUP;
            sc[buf][c] = p.scales[(size_t)row * groups + g];
            bi[buf][c] = p.biases[(size_t)row * groups + g];
        }
    };
#pragma unroll
    for (int k = 0; k < LMH_BUFS - 1; ++k) load_row(k, row0 + hw + 8 * k);   // in flight while the inputs are prepared

    // The row and the norm weight reach LDS in one round trip (16-byte loads where the row is
    // aligned); everything after reads LDS.  Read straight from memory, the strided sum below
    // would be a chain of dependent round trips at the start of every block.
    const bool vec = ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(p.norm_weight)) & 15u) == 0 &&
                     p.d % 8 == 0;
    if (vec) {
        for (uint32_t i = tid; i < p.d / 8; i += 256) {
            reinterpret_cast<uint4*>(hraw)[i] = reinterpret_cast<const uint4*>(h)[i];
            if (p.norm_weight) reinterpret_cast<uint4*>(wraw)[i] = reinterpret_cast<const uint4*>(p.norm_weight)[i];
        }
    } else {
        for (uint32_t i = tid; i < p.d; i += 256) {
            hraw[i] = h[i];
            if (p.norm_weight) wraw[i] = p.norm_weight[i];
        }
    }
    __syncthreads();
    float inv = 1.0f;
    if (p.norm_weight) {
        float acc = 0.0f;
        for (uint32_t i = lane; i < p.d; i += 64) {
            const float v = act_to_f32<ACT>(hraw[i]);
            acc = fmaf(v, v, acc);
        }
        inv = rms_inverse(rms_wave_sum(acc), p.d, p.eps);     // every wave for itself, the same bits
    }
    for (uint32_t i = tid; i < p.d; i += 256) {
        float v = act_to_f32<ACT>(hraw[i]);
        if (p.norm_weight)
            v = act_to_f32<ACT>(f32_to_act<ACT>(__fmul_rn(__fmul_rn(v, inv), bf16_to_f32(wraw[i]))));
        xn[i] = v;
    }
    __syncthreads();

    float xr[CPL][EPC], xs[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const uint32_t chunk = min(hl + 32 * c, chunks - 1);     // a lane without this chunk: a copy, never used
        const float4* src = reinterpret_cast<const float4*>(xn + chunk * EPC);
        xs[c] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPC / 4; ++e) {
            const float4 v = src[e];
            xr[c][4 * e] = v.x; xr[c][4 * e + 1] = v.y; xr[c][4 * e + 2] = v.z; xr[c][4 * e + 3] = v.w;
        }
#pragma unroll
        for (int e = 0; e < EPC; ++e) xs[c] = __fadd_rn(xs[c], xr[c][e]);
    }

    float best_v = -INFINITY;
    uint32_t best_i = 0xFFFFFFFFu;
    auto sum_row = [&](int buf, uint32_t row) {
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            // every lane does the arithmetic (a lane without this chunk on a copy of the last one)
            // and keeps its old sum by a select: a branch here would cut the step into pieces
            // that each wait for their loads
            float qf[EPC];
            unpack_chunk<BITS>(q[buf][c], qf);     // 4 bit: nibbles isolated as bytes, one conversion per code
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < EPC; ++e) dot = fmaf(qf[e], xr[c][e], dot);
            float next = fmaf(bf16_to_f32(sc[buf][c]), dot, acc);
            next = fmaf(bf16_to_f32(bi[buf][c]), xs[c], next);
            acc = hl + 32 * c < chunks ? next : acc;
        }
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) acc = __fadd_rn(acc, shfl_xor_f(acc, off));
        // rows ascend inside a half-wave: a later equal logit never replaces an earlier one
        if (row < row_end && isfinite(acc) && (best_i == 0xFFFFFFFFu || acc > best_v)) { best_v = acc; best_i = row; }
    };
    // Three register buffers: two rows of codes in flight while one is summed.  Every half-wave
    // takes the same number of steps and every step loads (a row past the end loads the last row
    // again and is not counted), so the loop unrolls into straight code in which the compiler
    // can count the loads in flight; with conditional loads it waited for all of them each step.
#pragma unroll
    for (int k = 0; k < LMH_STEPS; ++k) {
        if (k + LMH_BUFS - 1 < LMH_STEPS) load_row((k + LMH_BUFS - 1) % LMH_BUFS, row0 + hw + 8 * (k + LMH_BUFS - 1));
        sum_row(k % LMH_BUFS, row0 + hw + 8 * k);
    }
    float* res_v = lmh_lds + p.d;
    uint32_t* res_i = reinterpret_cast<uint32_t*>(lmh_lds + p.d + 8);
    if (hl == 0) { res_v[hw] = best_v; res_i[hw] = best_i; }
    __syncthreads();
    if (tid == 0) {
        float bv = -INFINITY;
        uint32_t bidx = 0xFFFFFFFFu;
        for (int k = 0; k < 8; ++k) {             // half-wave k owns rows row0 + k, + 8, ...: compare indices
            const float v = res_v[k];
            const uint32_t i = res_i[k];
            if (i != 0xFFFFFFFFu && (bidx == 0xFFFFFFFFu || v > bv || (v == bv && i < bidx))) { bv = v; bidx = i; }
        }
        p.summaries[(size_t)t * gridDim.x + blockIdx.x] = make_float2(bv, __uint_as_float(bidx));
    }
}

// The winner among the block results of one token (logit.metal:890-937): one block per token.
__global__ __launch_bounds__(256) void lm_head_reduce_kernel(const float2* summaries, uint32_t n_blocks,
                                                             uint32_t* out_tokens) {
    __shared__ float sv[256];
    __shared__ uint32_t si[256];
    const uint32_t t = blockIdx.x, tid = threadIdx.x;
    float bv = -INFINITY;
    uint32_t bidx = 0xFFFFFFFFu;
    for (uint32_t k = tid; k < n_blocks; k += 256) {
        const float2 s = summaries[(size_t)t * n_blocks + k];
        const uint32_t i = __float_as_uint(s.y);
        if (i != 0xFFFFFFFFu && (bidx == 0xFFFFFFFFu || s.x > bv || (s.x == bv && i < bidx))) { bv = s.x; bidx = i; }
    }
    sv[tid] = bv;
    si[tid] = bidx;
    __syncthreads();
    for (uint32_t w = 128; w >= 1; w >>= 1) {
        if (tid < w) {
            const float v = sv[tid + w];
            const uint32_t i = si[tid + w];
            if (i != 0xFFFFFFFFu && (si[tid] == 0xFFFFFFFFu || v > sv[tid] || (v == sv[tid] && i < si[tid]))) {
                sv[tid] = v;
                si[tid] = i;
            }
        }
        __syncthreads();
    }
    if (tid == 0) out_tokens[t] = si[0] == 0xFFFFFFFFu ? 0u : si[0];
}

}  // namespace nvmai
