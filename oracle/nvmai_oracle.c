/*
 * nvmai_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference's quantized-MoE hot path.  Only the
 * test-suite, the smoke check and the bench's cpu_baseline leg may use it.
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fPIC -shared (see Makefile).
 *
 * What pins each function (besides its own formula):
 *   bf16 / quantizer / dequantizer  reference property tests (flat group,
 *       full codebook, nibble order, one-step error bound) + brute-force
 *       nearest-code check                                   tests/test_oracle_quant.py
 *   expert offsets                  reference known answers (1,769,472 ...)  same file
 *   int4 GEMV                       bit-exact against the reference C file
 *       compiled from its own source (oracle/_ref), unfactored cross-check,
 *       bit-stream known answer                              tests/test_oracle_gemv_moe.py
 *   expert FFN / MoE layer          constant-blob known answer silu(2), float64
 *       dense recomputation, accumulate linearity            tests/test_oracle_gemv_moe.py
 *   router                          brute-force stable sort, near-tie cases of
 *       the reference tests                                  tests/test_oracle_gemv_moe.py
 *   pairs / grouping                full expected arrays of the reference tests
 *                                                             tests/test_oracle_prefill.py
 *   KV layout / quantizer           strides 1024/544/288; invariants (min->0,
 *       max->levels, flat->0) and brute-force nearest code.  No reference test
 *       holds KV codes, so the codes are pinned by the closed form only
 *       (PARITY UNPINNED against the reference).
 *   attention / RoPE                float64 textbook attention, split==single,
 *       geometry known answers, rope identity at position 0  tests/test_oracle_attention.py
 *   softmax / sampler               float64 softmax, tiled==single, generic ==
 *       top-64 token-for-token on the reference's LCG input, xorshift64*
 *       textbook values                                      tests/test_oracle_sampler.py
 *   Gumbel-max sampler              PARITY UNPINNED against the reference (it holds
 *       no vector and Metal's fast-math log is not reproducible): pinned by the
 *       published SplitMix64 constant, the closed form of the noise and the
 *       property that the draw follows p^(1/T)               tests/test_oracle_sampler.py
 *   RMSNorm                         float64 recomputation, the reference tests'
 *       constant-head known answer (every output 1), per-head isolation
 *                                                             tests/test_oracle_step.py
 *   elementwise helpers             PARITY UNPINNED against the reference (it holds no test
 *       for them): special values (sigmoid(0) = 1/2, silu(0) = 0, saturation) and float64
 *       recomputation; the add, split and concatenation are fixed by their definition
 *                                                             tests/test_oracle_step.py
 *   embedding lookup                the reference's bit-stream known answer
 *       (AffineQuantTests.swift:58-79), out-of-range token -> zeros, equals the
 *       dequantizer                                           tests/test_oracle_step.py
 *   greedy LM head                  the reference tests' known answers (target row,
 *       ties -> lowest index, all-NaN -> 0, strided hidden row), brute-force
 *       float64 argmax on well-separated rows                 tests/test_oracle_step.py
 *
 * Canonical summation order of the router logits ("half-wave order"):
 *   a row is cut into 16-byte chunks (16 codes at 8 bits, 32 codes at 4 bits,
 *   8 values for dense bf16).  32 virtual lanes; lane l owns chunks l, l+32,
 *   l+64, ...  Within a chunk the lane runs dot = fmaf(q, x, dot) and
 *   xs = xs + x in element order, then acc = fmaf(s, dot, acc);
 *   acc = fmaf(b, xs, acc) (dense: acc = fmaf(w, x, acc) per element).  The 32
 *   lane accumulators are summed by an xor butterfly with offsets 16, 8, 4, 2,
 *   1.  The reference fixes no order (moe.metal:205-213 uses simd_sum,
 *   prefill.metal:367-383 a sequential loop); routing indices are only
 *   reproducible against a stated order, and this is the one the HIP router
 *   implements.
 */
#include "nvmai_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* scalar conversions                                                        */
/* ------------------------------------------------------------------------ */

static inline uint32_t f32_bits(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float bits_f32(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* Quantization.swift:17-23: (bits + 0x7FFF + lsb) >> 16, wrapping, no NaN case */
uint16_t orc_bf16_bits(float x) {
    uint32_t bits = f32_bits(x);
    uint32_t lsb = (bits >> 16) & 1u;
    uint32_t rounded = (bits + 0x7FFFu + lsb) >> 16;
    return (uint16_t)rounded;
}

float orc_bf16_to_float(uint16_t bits) { return bits_f32(((uint32_t)bits) << 16); }

/* IEEE binary16 from binary32, round-to-nearest-even, subnormals kept. */
uint16_t orc_f16_bits(float x) {
    uint32_t u = f32_bits(x);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7FFFFFFFu;
    if (absu >= 0x7F800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absu > 0x7F800000u) ? 0x200u : 0u));
    }
    if (absu >= 0x477FF000u) {                       /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absu < 0x38800000u) {                        /* below 2^-14: subnormal */
        if (absu < 0x33000000u) return (uint16_t)sign;   /* < 2^-25 -> 0 */
        uint32_t mant = (absu & 0x007FFFFFu) | 0x00800000u;
        int exp = (int)(absu >> 23);                 /* biased */
        int shift = 126 - exp;                       /* 14..24 */
        /* value = mant * 2^(exp-150); half subnormal unit = 2^-24 */
        uint32_t q = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t exp = (absu >> 23) - 112u;              /* rebias 127 -> 15 */
    uint32_t mant = absu & 0x007FFFFFu;
    uint32_t h = (exp << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

float orc_f16_to_float(uint16_t bits) {
    uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
    uint32_t exp = (bits >> 10) & 0x1Fu;
    uint32_t mant = bits & 0x3FFu;
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        float v = (float)mant * 5.9604644775390625e-08f;  /* 2^-24 */
        return (sign ? -v : v);
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (mant << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

void orc_round_through_bf16(float *v, size_t n) {
    for (size_t i = 0; i < n; ++i) v[i] = orc_bf16_to_float(orc_bf16_bits(v[i]));
}

void orc_round_through_f16(float *v, size_t n) {
    for (size_t i = 0; i < n; ++i) v[i] = orc_f16_to_float(orc_f16_bits(v[i]));
}

/* ------------------------------------------------------------------------ */
/* test PRNGs                                                                */
/* ------------------------------------------------------------------------ */

uint64_t orc_splitmix64_next(orc_splitmix64 *s) {          /* SplitMix64.swift:11-17 */
    s->state += 0x9E3779B97F4A7C15ull;
    uint64_t z = s->state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

float orc_splitmix64_uniform(orc_splitmix64 *s, float lo, float hi) { /* :20-23 */
    float u = (float)(orc_splitmix64_next(s) >> 40) / 16777216.0f;
    return lo + (hi - lo) * u;
}

uint64_t orc_seedtree_key(uint64_t root, const char *label) {  /* SeedTree.swift:12-19 */
    uint64_t h = 0xCBF29CE484222325ull;
    for (const unsigned char *p = (const unsigned char *)label; *p; ++p) {
        h ^= (uint64_t)*p;
        h *= 0x100000001B3ull;
    }
    return root ^ h;
}

float orc_lcg_next(uint64_t *state, uint64_t inc) {        /* CPUExpertFFNTests.swift:18-23 */
    *state = *state * 6364136223846793005ull + inc;
    int32_t v = (int32_t)(uint32_t)(*state >> 33);
    return (float)v / (float)INT32_MAX;
}

/* ------------------------------------------------------------------------ */
/* affine quantizer                                                          */
/* ------------------------------------------------------------------------ */

/* Quantization.swift:59-99 / :144-175 */
void orc_quantize_affine(const float *w, size_t rows, size_t n, int bits,
                         uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    const int levels = (1 << bits) - 1;
    const size_t groups = n / ORC_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r) {
        const float *row = w + r * n;
        uint8_t *prow = packed + r * row_bytes;
        for (size_t g = 0; g < groups; ++g) {
            float wmin = INFINITY, wmax = -INFINITY;
            for (size_t k = 0; k < ORC_GROUP; ++k) {
                float v = row[g * ORC_GROUP + k];
                if (v < wmin) wmin = v;
                if (v > wmax) wmax = v;
            }
            float scale_f, bias_f;
            if (wmax == wmin) { scale_f = 1.0f; bias_f = wmin; }
            else { scale_f = (wmax - wmin) / (float)levels; bias_f = wmin; }
            uint16_t sb = orc_bf16_bits(scale_f), bb = orc_bf16_bits(bias_f);
            scales[r * groups + g] = sb;
            biases[r * groups + g] = bb;
            float scale = orc_bf16_to_float(sb), bias = orc_bf16_to_float(bb);
            float inv = (scale == 0.0f) ? 0.0f : 1.0f / scale;
            for (size_t k = 0; k < ORC_GROUP; ++k) {
                float t = (row[g * ORC_GROUP + k] - bias) * inv;
                float rt = roundf(t);                /* Swift .rounded(): half away */
                long q = (long)rt;
                if (q < 0) q = 0;
                if (q > levels) q = levels;
                size_t e = g * ORC_GROUP + k;
                if (bits == 8) {
                    prow[e] = (uint8_t)q;
                } else {
                    uint8_t nib = (uint8_t)q & 0x0F;
                    if ((e & 1) == 0) prow[e / 2] = (uint8_t)((prow[e / 2] & 0xF0) | nib);
                    else prow[e / 2] = (uint8_t)((prow[e / 2] & 0x0F) | (nib << 4));
                }
            }
        }
    }
}

static inline unsigned code_at(const uint8_t *row, size_t e, int bits) {
    if (bits == 8) return row[e];
    uint8_t b = row[e / 2];
    return (e & 1) ? (unsigned)(b >> 4) : (unsigned)(b & 0x0F);
}

void orc_dequantize_affine(const uint8_t *packed, const uint16_t *scales,
                           const uint16_t *biases, size_t rows, size_t n,
                           int bits, float *out) {
    const size_t groups = n / ORC_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r)
        for (size_t g = 0; g < groups; ++g) {
            float s = orc_bf16_to_float(scales[r * groups + g]);
            float b = orc_bf16_to_float(biases[r * groups + g]);
            for (size_t k = 0; k < ORC_GROUP; ++k) {
                size_t e = g * ORC_GROUP + k;
                out[r * n + e] = (float)code_at(packed + r * row_bytes, e, bits) * s + b;
            }
        }
}

void orc_unpack_codes(const uint8_t *packed, size_t count, int bits, uint8_t *codes) {
    for (size_t e = 0; e < count; ++e) codes[e] = (uint8_t)code_at(packed, e, bits);
}

/* ------------------------------------------------------------------------ */
/* expert blob                                                               */
/* ------------------------------------------------------------------------ */

/* CPUExpertFFN.swift:42-59 generalised from 4 bits to `bits` */
void orc_expert_offsets(size_t d, size_t f, int bits, uint32_t out[10]) {
    size_t gate_w = f * d * (size_t)bits / 8;
    size_t gate_meta = f * (d / ORC_GROUP) * 2;
    size_t down_w = d * f * (size_t)bits / 8;
    size_t down_meta = d * (f / ORC_GROUP) * 2;
    size_t o = 0;
    out[0] = (uint32_t)o; o += gate_w;
    out[1] = (uint32_t)o; o += gate_meta;
    out[2] = (uint32_t)o; o += gate_meta;
    out[3] = (uint32_t)o; o += gate_w;
    out[4] = (uint32_t)o; o += gate_meta;
    out[5] = (uint32_t)o; o += gate_meta;
    out[6] = (uint32_t)o; o += down_w;
    out[7] = (uint32_t)o; o += down_meta;
    out[8] = (uint32_t)o; o += down_meta;
    out[9] = (uint32_t)o;
}

void orc_pack_expert(const float *gate, const float *up, const float *down,
                     size_t d, size_t f, int bits, uint8_t *blob) {
    uint32_t off[10];
    orc_expert_offsets(d, f, bits, off);
    orc_quantize_affine(gate, f, d, bits, blob + off[0], (uint16_t *)(blob + off[1]),
                        (uint16_t *)(blob + off[2]));
    orc_quantize_affine(up, f, d, bits, blob + off[3], (uint16_t *)(blob + off[4]),
                        (uint16_t *)(blob + off[5]));
    orc_quantize_affine(down, d, f, bits, blob + off[6], (uint16_t *)(blob + off[7]),
                        (uint16_t *)(blob + off[8]));
}

/* ------------------------------------------------------------------------ */
/* GEMV                                                                      */
/* ------------------------------------------------------------------------ */

/* int4_affine_gemv.c:114-134: per group sequential dot and xsum, then
 * acc += s*dot + b*xsum (two products, one sum, one accumulate). */
void orc_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                          const uint16_t *biases, const float *x, size_t rows,
                          size_t n, float *out) {
    const size_t groups = n / ORC_GROUP;
    const size_t row_bytes = n / 2;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *wr = weights + r * row_bytes;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t *wg = wr + g * (ORC_GROUP / 2);
            const float *xg = x + g * ORC_GROUP;
            float dot = 0.0f, xsum = 0.0f;
            for (size_t k = 0; k < ORC_GROUP / 2; ++k) {
                float x0 = xg[2 * k], x1 = xg[2 * k + 1];
                dot += (float)(wg[k] & 0x0F) * x0 + (float)(wg[k] >> 4) * x1;
                xsum += x0 + x1;
            }
            acc += orc_bf16_to_float(scales[r * groups + g]) * dot
                 + orc_bf16_to_float(biases[r * groups + g]) * xsum;
        }
        out[r] = acc;
    }
}

void orc_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                     const uint16_t *biases, const float *x, size_t rows,
                     size_t n, int bits, float *out) {
    if (bits == 4) { orc_int4_affine_gemv(weights, scales, biases, x, rows, n, out); return; }
    const size_t groups = n / ORC_GROUP;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *wr = weights + r * n;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const uint8_t *wg = wr + g * ORC_GROUP;
            const float *xg = x + g * ORC_GROUP;
            float dot = 0.0f, xsum = 0.0f;
            /* same pairing as the 4-bit loop: two elements per step */
            for (size_t k = 0; k < ORC_GROUP / 2; ++k) {
                float x0 = xg[2 * k], x1 = xg[2 * k + 1];
                dot += (float)wg[2 * k] * x0 + (float)wg[2 * k + 1] * x1;
                xsum += x0 + x1;
            }
            acc += orc_bf16_to_float(scales[r * groups + g]) * dot
                 + orc_bf16_to_float(biases[r * groups + g]) * xsum;
        }
        out[r] = acc;
    }
}

void orc_affine_gemv_unfactored(const uint8_t *weights, const uint16_t *scales,
                                const uint16_t *biases, const float *x,
                                size_t rows, size_t n, int bits, float *out) {
    const size_t groups = n / ORC_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r) {
        float acc = 0.0f;
        for (size_t e = 0; e < n; ++e) {
            float s = orc_bf16_to_float(scales[r * groups + e / ORC_GROUP]);
            float b = orc_bf16_to_float(biases[r * groups + e / ORC_GROUP]);
            float wv = (float)code_at(weights + r * row_bytes, e, bits) * s + b;
            acc += wv * x[e];
        }
        out[r] = acc;
    }
}

/* ------------------------------------------------------------------------ */
/* expert FFN                                                                */
/* ------------------------------------------------------------------------ */

static inline float silu_f(float v) { return v / (1.0f + expf(-v)); }  /* CPUExpertFFN.swift:92-94 */

void orc_expert_ffn_accumulate(const uint8_t *blob, const uint32_t off[10],
                               int bits, const float *x, size_t d, size_t f,
                               float route_w, float *scratch, float *out) {
    float *gate_out = scratch, *up_out = scratch + f, *down_out = scratch + 2 * f;
    orc_affine_gemv(blob + off[0], (const uint16_t *)(blob + off[1]),
                    (const uint16_t *)(blob + off[2]), x, f, d, bits, gate_out);
    orc_affine_gemv(blob + off[3], (const uint16_t *)(blob + off[4]),
                    (const uint16_t *)(blob + off[5]), x, f, d, bits, up_out);
    for (size_t i = 0; i < f; ++i) gate_out[i] = silu_f(gate_out[i]) * up_out[i];
    orc_affine_gemv(blob + off[6], (const uint16_t *)(blob + off[7]),
                    (const uint16_t *)(blob + off[8]), gate_out, d, f, bits, down_out);
    for (size_t r = 0; r < d; ++r) out[r] += route_w * down_out[r];
}

/* ------------------------------------------------------------------------ */
/* router                                                                    */
/* ------------------------------------------------------------------------ */

void orc_router_logits(const void *weights, const uint16_t *scales,
                       const uint16_t *biases, int kind, const float *x,
                       const uint16_t *eff_scale, size_t num_experts, size_t d,
                       float *logits) {
    float *xe = (float *)malloc(d * sizeof(float));
    for (size_t i = 0; i < d; ++i)
        xe[i] = eff_scale ? x[i] * orc_bf16_to_float(eff_scale[i]) : x[i];
    const size_t per_chunk = (kind == 8) ? 16 : (kind == 4 ? 32 : 8);
    const size_t chunks = d / per_chunk;
    const size_t groups = d / ORC_GROUP;
    for (size_t e = 0; e < num_experts; ++e) {
        float lane[32];
        for (int l = 0; l < 32; ++l) {
            float acc = 0.0f;
            for (size_t c = (size_t)l; c < chunks; c += 32) {
                size_t base = c * per_chunk;
                if (kind == 16) {
                    const uint16_t *wr = (const uint16_t *)weights + e * d;
                    for (size_t k = 0; k < per_chunk; ++k)
                        acc = fmaf(orc_bf16_to_float(wr[base + k]), xe[base + k], acc);
                } else {
                    const uint8_t *wr = (const uint8_t *)weights + e * (d * (size_t)kind / 8);
                    size_t g = base / ORC_GROUP;
                    float s = orc_bf16_to_float(scales[e * groups + g]);
                    float b = orc_bf16_to_float(biases[e * groups + g]);
                    float dot = 0.0f, xs = 0.0f;
                    for (size_t k = 0; k < per_chunk; ++k) {
                        dot = fmaf((float)code_at(wr, base + k, kind), xe[base + k], dot);
                        xs = xs + xe[base + k];
                    }
                    acc = fmaf(s, dot, acc);
                    acc = fmaf(b, xs, acc);
                }
            }
            lane[l] = acc;
        }
        for (int off = 16; off >= 1; off >>= 1) {
            float next[32];
            for (int l = 0; l < 32; ++l) next[l] = lane[l] + lane[l ^ off];
            memcpy(lane, next, sizeof(lane));
        }
        logits[e] = lane[0];
    }
    free(xe);
}

/* moe.metal:233-285 generalised to k <= 64 (prefill.metal:386-434 is the same
 * insertion with a runtime k). */
void orc_router_topk(const float *logits, size_t num_experts, size_t k,
                     const uint16_t *per_expert_scale, uint32_t *out_idx,
                     uint16_t *out_w_f16) {
    uint32_t top_idx[64];
    float top_score[64];
    if (k > 64) k = 64;
    for (size_t i = 0; i < k; ++i) { top_idx[i] = 0; top_score[i] = -INFINITY; }
    for (size_t e = 0; e < num_experts; ++e) {
        float s = logits[e];
        if (s < top_score[k - 1]) continue;
        size_t pos = k;
        for (size_t i = 0; i < k; ++i) {
            if (s > top_score[i] || (s == top_score[i] && e < top_idx[i])) { pos = i; break; }
        }
        if (pos >= k) continue;
        for (size_t i = k - 1; i > pos; --i) {
            top_idx[i] = top_idx[i - 1];
            top_score[i] = top_score[i - 1];
        }
        top_idx[pos] = (uint32_t)e;
        top_score[pos] = s;
    }
    float max_s = top_score[0], sum_exp = 0.0f, exps[64];
    for (size_t i = 0; i < k; ++i) { exps[i] = expf(top_score[i] - max_s); sum_exp += exps[i]; }
    for (size_t i = 0; i < k; ++i) {
        float w = exps[i] / sum_exp;
        float gain = per_expert_scale ? orc_bf16_to_float(per_expert_scale[top_idx[i]]) : 1.0f;
        out_idx[i] = top_idx[i];
        out_w_f16[i] = orc_f16_bits(w * gain);
    }
}

void orc_moe_layer_forward(const orc_moe_layer *L, const float *x, size_t n_tokens,
                           uint32_t *out_idx, uint16_t *out_w_f16, float *y) {
    uint32_t off[10];
    orc_expert_offsets(L->d, L->f, L->bits, off);
    float *logits = (float *)malloc(L->num_experts * sizeof(float));
    float *scratch = (float *)malloc((2 * L->f + L->d) * sizeof(float));
    for (size_t t = 0; t < n_tokens; ++t) {
        const float *xt = x + t * L->d;
        float *yt = y + t * L->d;
        uint32_t *idx = out_idx + t * L->top_k;
        uint16_t *wts = out_w_f16 + t * L->top_k;
        orc_router_logits(L->router_w, L->router_s, L->router_b, L->router_kind, xt,
                          NULL, L->num_experts, L->d, logits);
        orc_router_topk(logits, L->num_experts, L->top_k, NULL, idx, wts);
        memset(yt, 0, L->d * sizeof(float));
        if (L->shared_blob) {
            orc_expert_ffn_accumulate(L->shared_blob, off, L->bits, xt, L->d, L->f, 1.0f,
                                      scratch, yt);
            if (L->gate_kind) {
                float g;
                orc_router_logits(L->gate_w, L->gate_s, L->gate_b, L->gate_kind, xt, NULL,
                                  1, L->d, &g);
                /* utility.metal:61-70: y / (1 + exp(-g)) */
                for (size_t r = 0; r < L->d; ++r) yt[r] = yt[r] / (1.0f + expf(-g));
            }
        }
        for (size_t s = 0; s < L->top_k; ++s)
            orc_expert_ffn_accumulate(L->experts[idx[s]], off, L->bits, xt, L->d, L->f,
                                      orc_f16_to_float(wts[s]), scratch, yt);
    }
    free(scratch);
    free(logits);
}

/* ------------------------------------------------------------------------ */
/* prefill pairs + grouping                                                  */
/* ------------------------------------------------------------------------ */

void orc_make_pairs(const uint32_t *idx, const uint16_t *w_f16, size_t tokens,
                    size_t k, orc_pair *pairs) {              /* PrefillRouter.swift:107-115 */
    for (size_t t = 0; t < tokens; ++t)
        for (size_t r = 0; r < k; ++r) {
            size_t i = t * k + r;
            pairs[i].token = (uint32_t)t;
            pairs[i].expert = idx[i];
            pairs[i].rank = (uint32_t)r;
            pairs[i].weight_bits = (uint32_t)w_f16[i];
        }
}

static const uint64_t *g_sort_keys;
static int pair_cmp(const void *pa, const void *pb) {         /* PrefillMoEGrouping.swift:140-149 */
    const orc_pair *a = (const orc_pair *)pa, *b = (const orc_pair *)pb;
    if (g_sort_keys) {
        uint64_t ka = g_sort_keys[a->expert], kb = g_sort_keys[b->expert];
        if (ka != kb) return ka < kb ? -1 : 1;
    }
    if (a->expert != b->expert) return a->expert < b->expert ? -1 : 1;
    if (a->token != b->token) return a->token < b->token ? -1 : 1;
    if (a->rank != b->rank) return a->rank < b->rank ? -1 : 1;
    return 0;
}

int orc_group_pairs(const orc_pair *pairs, size_t n_pairs, long query_count,
                    long top_k, long num_experts, long tile_expert_count,
                    const uint64_t *sort_keys, size_t n_sort_keys,
                    orc_pair *sorted, uint32_t *offsets, uint32_t *counts,
                    orc_group *groups, size_t *n_groups, orc_tile *tiles,
                    size_t *n_tiles) {
    if (query_count < 0) return ORC_GROUP_BAD_QUERY;          /* :99-110 */
    if (top_k <= 0) return ORC_GROUP_BAD_TOPK;
    if (num_experts <= 0) return ORC_GROUP_BAD_EXPERTS;
    if (tile_expert_count < 1 || tile_expert_count > 16) return ORC_GROUP_BAD_TILE;
    if (sort_keys && n_sort_keys != (size_t)num_experts) return ORC_GROUP_SORTKEY_COUNT;
    if (n_pairs != (size_t)(query_count * top_k)) return ORC_GROUP_PAIR_COUNT;
    uint8_t *seen = (uint8_t *)calloc(n_pairs ? n_pairs : 1, 1);
    for (size_t i = 0; i < n_pairs; ++i) {                    /* :121-137 */
        const orc_pair *p = &pairs[i];
        int rc = 0;
        if (p->token >= (uint32_t)query_count) rc = ORC_GROUP_TOKEN_RANGE;
        else if (p->rank >= (uint32_t)top_k) rc = ORC_GROUP_RANK_RANGE;
        else if (p->expert >= (uint32_t)num_experts) rc = ORC_GROUP_EXPERT_RANGE;
        else {
            size_t key = (size_t)p->token * (size_t)top_k + p->rank;
            if (seen[key]) rc = ORC_GROUP_DUPLICATE;
            seen[key] = 1;
        }
        if (rc) { free(seen); return rc; }
    }
    free(seen);
    memcpy(sorted, pairs, n_pairs * sizeof(orc_pair));
    g_sort_keys = sort_keys;
    qsort(sorted, n_pairs, sizeof(orc_pair), pair_cmp);   /* total order: stability moot */
    g_sort_keys = NULL;
    for (long e = 0; e < num_experts; ++e) { offsets[e] = 0xFFFFFFFFu; counts[e] = 0; }
    size_t ng = 0, i = 0;
    while (i < n_pairs) {                                     /* :156-169 */
        uint32_t e = sorted[i].expert;
        size_t start = i;
        while (i < n_pairs && sorted[i].expert == e) ++i;
        offsets[e] = (uint32_t)start;
        counts[e] = (uint32_t)(i - start);
        groups[ng].expert = e;
        groups[ng].pair_start = (uint32_t)start;
        groups[ng].pair_count = (uint32_t)(i - start);
        ++ng;
    }
    size_t nt = 0, gs = 0;
    while (gs < ng) {                                         /* :171-184 */
        size_t ge = gs + (size_t)tile_expert_count;
        if (ge > ng) ge = ng;
        tiles[nt].group_start = (uint32_t)gs;
        tiles[nt].group_count = (uint32_t)(ge - gs);
        tiles[nt].pair_start = groups[gs].pair_start;
        tiles[nt].pair_count = groups[ge - 1].pair_start + groups[ge - 1].pair_count
                             - groups[gs].pair_start;
        ++nt;
        gs = ge;
    }
    *n_groups = ng;
    *n_tiles = nt;
    return ORC_GROUP_OK;
}

void orc_prefill_moe(const uint8_t *const *experts, const uint32_t off[10],
                     int bits, const float *x, size_t tokens, size_t d, size_t f,
                     size_t k, const uint32_t *idx, const uint16_t *w_f16, float *h2) {
    float *scratch = (float *)malloc((2 * f + d) * sizeof(float));
    float *partial = (float *)malloc(d * sizeof(float));
    for (size_t t = 0; t < tokens; ++t) {
        float *out = h2 + t * d;
        memset(out, 0, d * sizeof(float));
        for (size_t r = 0; r < k; ++r) {                      /* prefill.metal:450-457 */
            memset(partial, 0, d * sizeof(float));
            orc_expert_ffn_accumulate(experts[idx[t * k + r]], off, bits, x + t * d, d, f,
                                      1.0f, scratch, partial);
            float w = orc_f16_to_float(w_f16[t * k + r]);
            for (size_t c = 0; c < d; ++c) out[c] = fmaf(w, partial[c], out[c]);
        }
    }
    free(partial);
    free(scratch);
}

/* ------------------------------------------------------------------------ */
/* KV cache                                                                  */
/* ------------------------------------------------------------------------ */

void orc_kv_row_layout(size_t elements, int bits, size_t *stride, size_t *value_bytes) {
    if (bits == 16) { *stride = elements * 2; *value_bytes = elements * 2; return; }
    size_t packed = (elements * (size_t)bits + 7) / 8;        /* KVCacheManager.swift:442-445 */
    size_t aligned = (packed + 1) & ~(size_t)1;
    size_t groups = (elements + ORC_GROUP - 1) / ORC_GROUP;
    *stride = aligned + groups * 2 * 2;
    *value_bytes = aligned;
}

static inline uint8_t kv_code(float v, float scale, float bias, float levels) {
    if (!(scale > 0.0f)) return 0;                            /* kv_cache_quantize.metal:56-59 */
    float t = (v - bias) / scale;
    if (t < 0.0f) t = 0.0f;
    if (t > levels) t = levels;
    return (uint8_t)roundf(t);
}

void orc_kv_quantize(const float *src, size_t src_stride, size_t tokens,
                     size_t elements, int bits, uint8_t *dst, size_t dst_stride,
                     size_t value_bytes) {
    const float levels = (bits == 4) ? 15.0f : 255.0f;
    const size_t groups = (elements + ORC_GROUP - 1) / ORC_GROUP;
    for (size_t t = 0; t < tokens; ++t) {
        const float *s = src + t * src_stride;
        uint8_t *row = dst + t * dst_stride;
        for (size_t g = 0; g < groups; ++g) {
            size_t lo = g * ORC_GROUP, hi = lo + ORC_GROUP;
            if (hi > elements) hi = elements;
            float mn = INFINITY, mx = -INFINITY;
            for (size_t i = lo; i < hi; ++i) {
                mn = fminf(mn, s[i]);
                mx = fmaxf(mx, s[i]);
            }
            float bias = mn;
            float scale = (mx > mn) ? (mx - mn) / levels : 0.0f;
            uint16_t sb = orc_f16_bits(scale), bb = orc_f16_bits(bias);
            memcpy(row + value_bytes + 2 * g, &sb, 2);
            memcpy(row + value_bytes + 2 * groups + 2 * g, &bb, 2);
            for (size_t i = lo; i < hi; ++i) {
                uint8_t c = kv_code(s[i], scale, bias, levels);
                if (bits == 8) row[i] = c;
                else if ((i & 1) == 0) {
                    uint8_t high = (i + 1 < elements) ? kv_code(s[i + 1], scale, bias, levels) : 0;
                    /* i+1 is in the same group because groups are even-sized */
                    row[i / 2] = (uint8_t)(c | (high << 4));
                }
            }
        }
    }
}

void orc_kv_dequant_row(const uint8_t *row, size_t elements, int bits,
                        size_t value_bytes, float *out) {      /* attention.metal:101-116 */
    const size_t groups = (elements + ORC_GROUP - 1) / ORC_GROUP;
    for (size_t i = 0; i < elements; ++i) {
        uint16_t sb, bb;
        size_t g = i / ORC_GROUP;
        memcpy(&sb, row + value_bytes + 2 * g, 2);
        memcpy(&bb, row + value_bytes + 2 * groups + 2 * g, 2);
        out[i] = (float)code_at(row, i, bits) * orc_f16_to_float(sb) + orc_f16_to_float(bb);
    }
}

void orc_rope_neox_subdim(float *data, size_t tokens, size_t heads, size_t head_dim,
                          size_t rotary_dim, const uint32_t *positions, float theta) {
    const size_t half_rot = rotary_dim / 2;                   /* rope.metal:94-101 */
    for (size_t t = 0; t < tokens; ++t)
        for (size_t h = 0; h < heads; ++h) {
            float *head = data + (t * heads + h) * head_dim;
            for (size_t p = 0; p < half_rot; ++p) {           /* rope.metal:32-50 */
                float exponent = -(float)(2u * (uint32_t)p) / (float)(uint32_t)rotary_dim;
                float angle = (float)positions[t] * powf(theta, exponent);
                float c = cosf(angle), s = sinf(angle);
                float x0 = head[p], x1 = head[half_rot + p];
                head[p] = x0 * c - x1 * s;
                head[half_rot + p] = x0 * s + x1 * c;
            }
        }
}

void orc_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                        uint32_t kv_start, int prefer_gqa_swa, uint32_t *eff_len,
                        uint32_t *num_chunks, uint32_t *chunk_len,
                        uint32_t *partial_groups) {           /* Attention.swift:142-167 */
    const long default_full = 16, default_gqa_swa = 8, max_chunks = 64;  /* Attention.swift:51-54 */
    long q_per_kv = num_q_heads / num_kv_heads;
    int use_gqa = prefer_gqa_swa && q_per_kv <= 2;
    long eff = (long)seq_len - (long)kv_start;
    long e1 = eff > 1 ? eff : 1;
    long def = use_gqa ? default_gqa_swa : default_full;
    long base = def < max_chunks ? def : max_chunks;
    if (e1 < base) base = e1;
    if (base < 1) base = 1;
    long nc = base;
    if (use_gqa) {
        long alt = base * q_per_kv;
        if (alt > max_chunks) alt = max_chunks;
        if (alt > nc) nc = alt;
    }
    *eff_len = (uint32_t)eff;
    *num_chunks = (uint32_t)nc;
    *chunk_len = (uint32_t)((e1 + nc - 1) / nc);
    *partial_groups = (uint32_t)((use_gqa ? num_kv_heads : num_q_heads) * nc);
}

static void kv_row_as_float(const void *base, int kv_bits, size_t stride, size_t value_bytes,
                            size_t elements, size_t p, float *tmp, const float **out) {
    if (kv_bits == 32) { *out = (const float *)base + p * elements; return; }
    orc_kv_dequant_row((const uint8_t *)base + p * stride, elements, kv_bits, value_bytes, tmp);
    *out = tmp;
}

void orc_attention_decode(const float *q, const void *k, const void *v, int kv_bits,
                          size_t stride, size_t value_bytes, size_t num_q_heads,
                          size_t num_kv_heads, size_t head_dim, size_t seq_len,
                          size_t kv_start, float scale, size_t num_chunks,
                          size_t chunk_len, float *out) {
    const size_t elements = num_kv_heads * head_dim;
    const size_t len = seq_len > kv_start ? seq_len - kv_start : 0;
    float *kt = (float *)malloc(elements * sizeof(float));
    float *vt = (float *)malloc(elements * sizeof(float));
    const size_t nc = num_chunks ? num_chunks : 1;
    const size_t cl = num_chunks ? chunk_len : (len ? len : 1);
    /* per (head, chunk) online-softmax state: attention.metal:212-251 */
    float *m = (float *)malloc(num_q_heads * nc * sizeof(float));
    float *dsum = (float *)malloc(num_q_heads * nc * sizeof(float));
    float *o = (float *)calloc(num_q_heads * nc * head_dim, sizeof(float));
    for (size_t i = 0; i < num_q_heads * nc; ++i) { m[i] = -INFINITY; dsum[i] = 0.0f; }
    for (size_t c = 0; c < nc; ++c) {
        size_t p0 = kv_start + c * cl, p1 = p0 + cl;
        if (p1 > seq_len) p1 = seq_len;
        for (size_t p = p0; p < p1; ++p) {
            const float *kr, *vr;
            kv_row_as_float(k, kv_bits, stride, value_bytes, elements, p, kt, &kr);
            kv_row_as_float(v, kv_bits, stride, value_bytes, elements, p, vt, &vr);
            for (size_t h = 0; h < num_q_heads; ++h) {
                size_t kvh = h / (num_q_heads / num_kv_heads);
                const float *qh = q + h * head_dim;
                float s = 0.0f;
                for (size_t i = 0; i < head_dim; ++i) s = fmaf(qh[i], kr[kvh * head_dim + i], s);
                s *= scale;
                size_t st = h * nc + c;
                float m_new = fmaxf(m[st], s);
                float alpha = expf(m[st] - m_new);
                float pe = expf(s - m_new);
                dsum[st] = dsum[st] * alpha + pe;
                float *oh = o + st * head_dim;
                for (size_t i = 0; i < head_dim; ++i)
                    oh[i] = oh[i] * alpha + pe * vr[kvh * head_dim + i];
                m[st] = m_new;
            }
        }
    }
    for (size_t h = 0; h < num_q_heads; ++h) {                /* attention.metal:388-429 */
        float mg = -INFINITY;
        for (size_t c = 0; c < nc; ++c) mg = fmaxf(mg, m[h * nc + c]);
        float *oh = out + h * head_dim;
        if (mg == -INFINITY) { memset(oh, 0, head_dim * sizeof(float)); continue; }
        float D = 0.0f;
        for (size_t c = 0; c < nc; ++c) D += dsum[h * nc + c] * expf(m[h * nc + c] - mg);
        float inv = D > 0.0f ? 1.0f / D : 0.0f;
        for (size_t i = 0; i < head_dim; ++i) {
            float acc = 0.0f;
            for (size_t c = 0; c < nc; ++c)
                acc += o[(h * nc + c) * head_dim + i] * expf(m[h * nc + c] - mg);
            oh[i] = acc * inv;
        }
    }
    free(o); free(dsum); free(m); free(vt); free(kt);
}

void orc_attention_prefill_causal(const float *q, size_t q_stride, const void *k, const void *v,
                                  int kv_bits, size_t stride, size_t value_bytes,
                                  size_t num_q_heads, size_t num_kv_heads, size_t head_dim,
                                  size_t start, size_t count, size_t kv_valid, size_t window,
                                  size_t ring, float scale, float *out, size_t out_stride) {
    const size_t elements = num_kv_heads * head_dim;
    const size_t q_per_kv = num_q_heads / num_kv_heads;
    float *kt = (float *)malloc(elements * sizeof(float));
    float *vt = (float *)malloc(elements * sizeof(float));
    float *row_max = (float *)malloc(num_q_heads * sizeof(float));
    float *row_sum = (float *)malloc(num_q_heads * sizeof(float));
    float *acc = (float *)malloc(num_q_heads * head_dim * sizeof(float));
    for (size_t t = 0; t < count; ++t) {
        const size_t abs_q = start + t;
        const size_t first = (window != 0 && abs_q + 1 > window) ? abs_q + 1 - window : 0;
        const size_t last = kv_valid < abs_q + 1 ? kv_valid : abs_q + 1;
        for (size_t h = 0; h < num_q_heads; ++h) { row_max[h] = -INFINITY; row_sum[h] = 0.0f; }
        memset(acc, 0, num_q_heads * head_dim * sizeof(float));
        for (size_t key = first; key < last; ++key) {
            const size_t slot = ring ? key % ring : key;
            const float *kr, *vr;
            kv_row_as_float(k, kv_bits, stride, value_bytes, elements, slot, kt, &kr);
            kv_row_as_float(v, kv_bits, stride, value_bytes, elements, slot, vt, &vr);
            for (size_t h = 0; h < num_q_heads; ++h) {
                const size_t kvh = h / q_per_kv;
                const float *qh = q + t * q_stride + h * head_dim;
                float s = 0.0f;
                for (size_t i = 0; i < head_dim; ++i) s = fmaf(qh[i], kr[kvh * head_dim + i], s);
                s *= scale;
                const float new_max = fmaxf(row_max[h], s);
                const float old_scale = row_sum[h] > 0.0f ? expf(row_max[h] - new_max) : 0.0f;
                const float new_scale = expf(s - new_max);
                float *a = acc + h * head_dim;
                for (size_t i = 0; i < head_dim; ++i)
                    a[i] = fmaf(new_scale, vr[kvh * head_dim + i], a[i] * old_scale);
                row_sum[h] = row_sum[h] * old_scale + new_scale;
                row_max[h] = new_max;
            }
        }
        for (size_t h = 0; h < num_q_heads; ++h)
            for (size_t i = 0; i < head_dim; ++i)
                out[t * out_stride + h * head_dim + i] =
                    row_sum[h] > 0.0f ? acc[h * head_dim + i] / row_sum[h] : 0.0f;
    }
    free(acc); free(row_sum); free(row_max); free(vt); free(kt);
}

/* ------------------------------------------------------------------------ */
/* softmax + sampler                                                         */
/* ------------------------------------------------------------------------ */
/* rest of the decode step: RMSNorm, embedding lookup, greedy LM head         */
/* ------------------------------------------------------------------------ */

/* rmsnorm.metal:31-62 (inv = rsqrt(mean(x^2) + eps)), :83-87 (y = x * inv * w, left to right),
 * :166-170 (no weight); rows = heads for the per-head kernels (:101-148).  The reference sums
 * with a 256-thread block reduction whose order Metal does not fix; the order stated here is
 * the one the HIP kernel implements, so that results can be compared bit for bit: 64 virtual
 * lanes, lane l runs acc = fmaf(x, x, acc) over the elements l, l + 64, ... in ascending
 * order, the 64 accumulators are summed by an xor butterfly with offsets 32, 16, 8, 4, 2, 1;
 * mean = sum / d, inv = 1 / sqrtf(mean + eps), every operation rounded once.  weight: BF16
 * bits or NULL.  out is NOT rounded to the activation type. */
void orc_rmsnorm(const float *x, size_t x_stride, const uint16_t *weight_bf16, size_t rows,
                 size_t d, float eps, float *out, size_t out_stride) {
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * x_stride;
        float lane[64];
        for (int l = 0; l < 64; ++l) {
            float acc = 0.0f;
            for (size_t i = (size_t)l; i < d; i += 64) acc = fmaf(xr[i], xr[i], acc);
            lane[l] = acc;
        }
        for (int off = 32; off >= 1; off >>= 1) {
            float next[64];
            for (int l = 0; l < 64; ++l) next[l] = lane[l] + lane[l ^ off];
            memcpy(lane, next, sizeof(lane));
        }
        const float mean = lane[0] / (float)d;
        const float inv = 1.0f / sqrtf(mean + eps);
        for (size_t i = 0; i < d; ++i) {
            float v = xr[i] * inv;
            if (weight_bf16) v = v * orc_bf16_to_float(weight_bf16[i]);
            out[r * out_stride + i] = v;
        }
    }
}

/* utility.metal:32-45, 47-58, 60-72, 95-104: op 0 silu(a) * b, 1 a * sigmoid(b[i]) written as
 * a / (1 + exp(-b)), 2 the same with b[0], 3 a + b; fp32, each operation rounded once.  out is
 * NOT rounded to the activation type. */
void orc_elementwise(int op, const float *a, const float *b, size_t count, float *out) {
    for (size_t i = 0; i < count; ++i) {
        const float x = a[i], y = b[op == 2 ? 0 : i];
        if (op == 0) out[i] = (x / (1.0f + expf(-x))) * y;
        else if (op == 3) out[i] = x + y;
        else out[i] = x / (1.0f + expf(-y));
    }
}

/* dequant_int4.metal:63-91 for 4- and 8-bit tables (AffineQuantEmbeddingLookup):
 * out[i] = (float(q) * s + b) * out_scale, two roundings then the scale; a token id at or
 * past vocab gives a row of zeros (:77-80).  out is NOT rounded to the activation type. */
void orc_embed_lookup(const uint8_t *table, const uint16_t *scales, const uint16_t *biases,
                      int bits, uint32_t token, size_t vocab, size_t d, float out_scale,
                      float *out) {
    if (token >= vocab) { for (size_t i = 0; i < d; ++i) out[i] = 0.0f; return; }
    const size_t groups = d / ORC_GROUP;
    const uint8_t *row = table + (size_t)token * (d * (size_t)bits / 8);
    for (size_t i = 0; i < d; ++i) {
        const float s = orc_bf16_to_float(scales[token * groups + i / ORC_GROUP]);
        const float b = orc_bf16_to_float(biases[token * groups + i / ORC_GROUP]);
        const float w = (float)code_at(row, i, bits) * s + b;
        out[i] = w * out_scale;
    }
}

/* LMHeadChainInt4.encodeGreedyDecode (LMHeadChainInt4.swift:58-130): RMSNorm with a BF16
 * weight (norm_weight NULL: the hidden row is used as it is), the normed row rounded to the
 * activation type (act 0 = bf16, 1 = fp16; the reference stores it as half), one logit per
 * vocabulary row, argmax over the FINITE logits with ties to the lower index, 0 when there
 * is none (logit.metal:855-861, 925-934).  The reference's per-row sum is a 32-lane simd_sum
 * whose order Metal does not fix; the logits here are taken in the router's canonical
 * half-wave order (above), which the HIP kernel implements, so the token is reproducible. */
uint32_t orc_lm_head_greedy(const float *hidden, const uint16_t *norm_weight_bf16,
                            const uint8_t *weights, const uint16_t *scales,
                            const uint16_t *biases, int bits, size_t d, size_t vocab,
                            float eps, int act, float *logits_out) {
    float *xn = (float *)malloc(d * sizeof(float));
    if (norm_weight_bf16) orc_rmsnorm(hidden, d, norm_weight_bf16, 1, d, eps, xn, d);
    else memcpy(xn, hidden, d * sizeof(float));
    if (act == 0) orc_round_through_bf16(xn, d); else orc_round_through_f16(xn, d);
    float *logits = logits_out ? logits_out : (float *)malloc(vocab * sizeof(float));
    orc_router_logits(weights, scales, biases, bits, xn, NULL, vocab, d, logits);
    float best_v = -INFINITY;
    uint32_t best_i = 0xFFFFFFFFu;
    for (size_t r = 0; r < vocab; ++r) {
        const float z = logits[r];
        if (!isfinite(z)) continue;
        if (best_i == 0xFFFFFFFFu || z > best_v) { best_v = z; best_i = (uint32_t)r; }
    }
    if (!logits_out) free(logits);
    free(xn);
    return best_i == 0xFFFFFFFFu ? 0u : best_i;
}

/* ------------------------------------------------------------------------ */

static inline float softcap_value(float z, float softcap) {   /* logit.metal:42-49 */
    if (softcap <= 0.0f) return z;
    return softcap * tanhf(z / softcap);
}

void orc_softmax_f16(const float *logits, size_t v, float softcap, uint16_t *probs_f16) {
    float m = -INFINITY;
    for (size_t i = 0; i < v; ++i) m = fmaxf(m, softcap_value(logits[i], softcap));
    float d = 0.0f;
    for (size_t i = 0; i < v; ++i) d += expf(softcap_value(logits[i], softcap) - m);
    float inv = d > 0.0f ? 1.0f / d : 0.0f;
    for (size_t i = 0; i < v; ++i)
        probs_f16[i] = orc_f16_bits(expf(softcap_value(logits[i], softcap) - m) * inv);
}

void orc_softmax_tiled_f16(const float *logits, size_t v, float softcap,
                           uint16_t *probs_f16) {             /* logit.metal:152-257 */
    const size_t tile = 4096;
    const size_t tiles = (v + tile - 1) / tile;
    float m = -INFINITY, d = 0.0f;
    for (size_t t = 0; t < tiles; ++t) {
        size_t lo = t * tile, hi = lo + tile;
        if (hi > v) hi = v;
        float tm = -INFINITY, td = 0.0f;
        for (size_t i = lo; i < hi; ++i) {                    /* stage 1 recurrence :176-182 */
            float z = softcap_value(logits[i], softcap);
            float mn = fmaxf(tm, z);
            float sc = (tm == -INFINITY) ? 0.0f : expf(tm - mn);
            td = td * sc + expf(z - mn);
            tm = mn;
        }
        float mn = fmaxf(m, tm);                              /* merge :217-225 */
        float sc = (m == -INFINITY) ? 0.0f : expf(m - mn);
        float contrib = (tm == -INFINITY) ? 0.0f : td * expf(tm - mn);
        d = d * sc + contrib;
        m = mn;
    }
    float inv = d > 0.0f ? 1.0f / d : 0.0f;
    for (size_t i = 0; i < v; ++i)                            /* normalize :246-257 */
        probs_f16[i] = orc_f16_bits(expf(softcap_value(logits[i], softcap) - m) * inv);
}

uint64_t orc_xorshift64star(uint64_t *s) {
    *s ^= *s << 13;
    *s ^= *s >> 7;
    *s ^= *s << 17;
    return *s * 2685821657736338717ull;
}

float orc_uniform01(uint64_t *s) {
    uint32_t bits = (uint32_t)(orc_xorshift64star(s) >> 40);
    return (float)bits * (1.0f / 16777216.0f);
}

uint64_t orc_seed_for(uint64_t seed, int64_t position) {
    uint64_t z = seed + (uint64_t)position + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return z == 0 ? 0x9E3779B97F4A7C15ull : z;
}

/* shared tail of both samplers: logit.metal:517-571 / :704-757 */
static uint32_t sample_tail(float *val, const uint32_t *idx, uint32_t kept,
                            float temperature, float top_p, uint64_t seed,
                            uint32_t fallback) {
    if (top_p > 0.0f && top_p < 1.0f) {
        float cum = 0.0f;
        uint32_t cut = kept;
        for (uint32_t i = 0; i < kept; ++i) {
            cum += val[i];
            if (cum >= top_p) { cut = i + 1; break; }
        }
        kept = cut;
    }
    float inv_t = 1.0f / temperature;
    if (temperature != 1.0f)
        for (uint32_t i = 0; i < kept; ++i) val[i] = powf(val[i], inv_t);
    float surviving = 0.0f;
    for (uint32_t i = 0; i < kept; ++i) surviving += val[i];
    uint64_t rng = seed;
    (void)orc_xorshift64star(&rng);
    float u = orc_uniform01(&rng) * surviving;
    float run = 0.0f;
    uint32_t picked = fallback;
    for (uint32_t i = 0; i < kept; ++i) {
        run += val[i];
        if (u <= run) { picked = idx[i]; break; }
    }
    return picked;
}

uint32_t orc_sample_generic(const uint16_t *probs_f16, size_t v, float temperature,
                            uint32_t top_k, float top_p, uint64_t seed) {
    if (temperature <= 0.0f) {                                /* logit.metal:340-382 */
        float best = -INFINITY;
        uint32_t bi = 0xFFFFFFFFu;
        for (size_t i = 0; i < v; ++i) {
            float p = orc_f16_to_float(probs_f16[i]);
            if (p > best) { best = p; bi = (uint32_t)i; }
        }
        /* no value above -inf (all NaN or -inf): every lane of the reference keeps best_i = 0 */
        return bi == 0xFFFFFFFFu ? 0u : bi;
    }
    size_t k = (top_k == 0) ? v : top_k;                      /* :464-467 */
    if (k > 256) k = 256;
    if (k > v) k = v;
    float val[256];
    uint32_t idx[256];
    uint32_t count = 0;
    uint8_t *claimed = (uint8_t *)calloc(v, 1);
    for (size_t slot = 0; slot < k; ++slot) {                 /* :479-517 */
        float best = -INFINITY;
        uint32_t bi = 0xFFFFFFFFu;
        for (size_t i = 0; i < v; ++i) {
            if (claimed[i]) continue;
            float p = orc_f16_to_float(probs_f16[i]);
            if (p > best) { best = p; bi = (uint32_t)i; }
        }
        val[slot] = best;
        idx[slot] = bi;
        count = (uint32_t)slot + 1;
        if (bi != 0xFFFFFFFFu) claimed[bi] = 1;
    }
    free(claimed);
    uint32_t kept = 0;
    while (kept < count && idx[kept] < v && isfinite(val[kept])) kept++;
    return sample_tail(val, idx, kept, temperature, top_p, seed, kept > 0 ? idx[0] : 0u);
}

/* Gumbel-max draw the reference takes when neither top-k nor top-p is set
 * (logit.metal:296-313, 391-429): argmax_i(log(p_i)/T + g_i), g_i = -log(-log(u_i)), u_i from a
 * counter-based SplitMix64 of (seed, position, i); zero and negative probabilities are skipped;
 * highest score wins, lowest index among equals; nothing eligible -> token 0.  The logarithms
 * are taken in double and rounded to float, one rounding per step, so that a restatement on
 * another device can reproduce the scores bit for bit (Metal's fast-math log cannot be). */
static uint64_t lmhead_splitmix64(uint64_t x) {               /* logit.metal:296-301 */
    x = x + 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

float orc_gumbel_for(uint64_t seed, uint32_t position, uint32_t row) {   /* :303-313 */
    uint64_t key = seed ^ ((uint64_t)position * 0xD2B74407B1CE6E93ull) ^ (uint64_t)row;
    uint32_t bits = (uint32_t)(lmhead_splitmix64(key) >> 40);
    float u = ((float)bits + 0.5f) * (1.0f / 16777216.0f);
    float inner = (float)log((double)u);
    return -(float)log((double)(-inner));
}

uint32_t orc_sample_gumbel(const uint16_t *probs_f16, size_t v, float temperature,
                           uint64_t seed, uint32_t position) {
    float inv_t = 1.0f / temperature;
    float best = -INFINITY;
    uint32_t bi = 0xFFFFFFFFu;
    for (size_t i = 0; i < v; ++i) {
        float p = orc_f16_to_float(probs_f16[i]);
        if (!(p > 0.0f)) continue;
        float s = inv_t * (float)log((double)p) + orc_gumbel_for(seed, position, (uint32_t)i);
        if (s > best) { best = s; bi = (uint32_t)i; }
    }
    return bi == 0xFFFFFFFFu ? 0u : bi;
}

/* The kernel's choice of path (logit.metal:340, 391, 431). */
uint32_t orc_sample(const uint16_t *probs_f16, size_t v, float temperature, uint32_t top_k,
                    float top_p, uint64_t seed, uint32_t position) {
    if (temperature > 0.0f && top_k == 0u && (top_p <= 0.0f || top_p >= 1.0f))
        return orc_sample_gumbel(probs_f16, v, temperature, seed, position);
    return orc_sample_generic(probs_f16, v, temperature, top_k, top_p, seed);
}

typedef struct { float v; uint32_t i; } cand;
static int cand_cmp(const void *pa, const void *pb) {         /* logit.metal:590-594 */
    const cand *a = (const cand *)pa, *b = (const cand *)pb;
    if (a->v > b->v) return -1;
    if (a->v < b->v) return 1;
    if (a->i < b->i) return -1;
    if (a->i > b->i) return 1;
    return 0;
}

/* One stage: sort each 1024-entry tile by (value desc, index asc), keep 64. */
static size_t topk64_stage(const cand *in, size_t count, cand *out) {
    size_t tiles = (count + 1023) / 1024;
    cand tile[1024];
    for (size_t t = 0; t < tiles; ++t) {
        for (size_t i = 0; i < 1024; ++i) {
            size_t src = t * 1024 + i;
            if (src < count) tile[i] = in[src];
            else { tile[i].v = -INFINITY; tile[i].i = 0xFFFFFFFFu; }
        }
        qsort(tile, 1024, sizeof(cand), cand_cmp);
        memcpy(out + t * 64, tile, 64 * sizeof(cand));
    }
    return tiles * 64;
}

uint32_t orc_sample_topk64(const uint16_t *probs_f16, size_t v, float temperature,
                           float top_p, uint64_t seed, uint32_t top_k,
                           uint32_t *top64_idx, float *top64_val) {
    cand *a = (cand *)malloc(v * sizeof(cand));
    for (size_t i = 0; i < v; ++i) { a[i].v = orc_f16_to_float(probs_f16[i]); a[i].i = (uint32_t)i; }
    size_t n1 = ((v + 1023) / 1024) * 64;
    cand *s1 = (cand *)malloc(n1 * sizeof(cand));
    n1 = topk64_stage(a, v, s1);                              /* stage1 :628-654 */
    size_t n2 = ((n1 + 1023) / 1024) * 64;
    cand *s2 = (cand *)malloc(n2 * sizeof(cand));
    n2 = topk64_stage(s1, n1, s2);                            /* reduce :656-682 */
    cand fin[1024];
    for (size_t i = 0; i < 1024; ++i) {                       /* final :684-703; needs n2 <= 1024 */
        if (i < n2) fin[i] = s2[i];
        else { fin[i].v = -INFINITY; fin[i].i = 0xFFFFFFFFu; }
    }
    qsort(fin, 1024, sizeof(cand), cand_cmp);
    free(s2); free(s1); free(a);
    float val[64];
    uint32_t idx[64];
    for (int i = 0; i < 64; ++i) { val[i] = fin[i].v; idx[i] = fin[i].i; }
    if (top64_idx) memcpy(top64_idx, idx, sizeof(idx));
    if (top64_val) memcpy(top64_val, val, sizeof(val));
    uint32_t kept = 0;
    while (kept < 64 && idx[kept] != 0xFFFFFFFFu && isfinite(val[kept])) kept++;
    uint32_t cap = top_k > 1 ? top_k : 1;
    if (kept > cap) kept = cap;
    return sample_tail(val, idx, kept, temperature, top_p, seed, idx[0]);
}

/* ------------------------------------------------------------------------ */
/* gated DeltaNet linear attention                                            */
/* ------------------------------------------------------------------------ */

static float round_act(float v, int act) {
    return act == 0 ? orc_bf16_to_float(orc_bf16_bits(v)) : orc_f16_to_float(orc_f16_bits(v));
}
static float gdn_silu(float x) { return x / (1.0f + expf(-x)); }                 /* gdn.metal:71-73 */
static float gdn_softplus(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }   /* :75-79 */

/* GDNReference.step (GDNReference.swift:41-114), the CPU model of one token through the kernels of
 * gdn.metal:241-271 (conv + SiLU, tail shift), :386-441 (q / k norm with the folded scales 1 / Dk and
 * 1 / sqrt(Dk)), :443-508 (gated delta rule) and :589-642 (gated output norm), with the reference's
 * rounding points: conv output, normed q / k and y are rounded to the activation type (act 0 = bf16,
 * 1 = fp16, the reference's), the tail keeps the raw row rounded to it, the state stays fp32.
 *   qkv_raw [C], a, b [Hv], z [Hv * Dv]: projection outputs (activation values as floats)
 *   conv_w [C, taps], a_log, dt_bias [Hv], norm_w [Dv]: BF16 bits
 *   tail [(taps - 1), C] and state [Hv, Dv, Dk] are updated in place; out [Hv * Dv] is NOT rounded. */
void orc_gdn_step(const float *qkv_raw, const float *a, const float *b, const float *z,
                  const uint16_t *conv_w, const uint16_t *a_log, const uint16_t *dt_bias,
                  const uint16_t *norm_w, size_t k_heads, size_t v_heads, size_t dk, size_t dv,
                  size_t taps, int act, float *tail, float *state, float *out) {
    const size_t C = 2 * k_heads * dk + v_heads * dv, hist = taps - 1;
    float *conv = (float *)malloc(C * sizeof(float));
    float *normed = (float *)malloc(C * sizeof(float));
    float *y = (float *)malloc(v_heads * dv * sizeof(float));
    for (size_t ch = 0; ch < C; ++ch) {                       /* GDNReference.swift:50-58 */
        float acc = qkv_raw[ch] * orc_bf16_to_float(conv_w[ch * taps + hist]);
        for (size_t j = 0; j < hist; ++j) acc += tail[j * C + ch] * orc_bf16_to_float(conv_w[ch * taps + j]);
        conv[ch] = round_act(gdn_silu(acc), act);
    }
    for (size_t j = 0; j + 1 < hist; ++j) memcpy(tail + j * C, tail + (j + 1) * C, C * sizeof(float));
    if (hist) for (size_t ch = 0; ch < C; ++ch) tail[(hist - 1) * C + ch] = round_act(qkv_raw[ch], act);
    memcpy(normed, conv, C * sizeof(float));
    for (size_t hi = 0; hi < 2 * k_heads; ++hi) {             /* :62-74 */
        const int is_q = hi < k_heads;
        const size_t base = (is_q ? 0 : k_heads * dk) + (is_q ? hi : hi - k_heads) * dk;
        float sumsq = 0.0f;
        for (size_t i = 0; i < dk; ++i) sumsq += conv[base + i] * conv[base + i];
        const float inv = 1.0f / sqrtf(sumsq / (float)dk + 1e-6f);
        const float scale = is_q ? 1.0f / (float)dk : 1.0f / sqrtf((float)dk);
        for (size_t i = 0; i < dk; ++i) normed[base + i] = round_act(conv[base + i] * inv * scale, act);
    }
    for (size_t h = 0; h < v_heads; ++h) {                    /* :77-99 */
        const size_t hk = h / (v_heads / k_heads);
        const float *q = normed + hk * dk, *k = normed + k_heads * dk + hk * dk;
        const float *v = normed + 2 * k_heads * dk + h * dv;
        const float g = expf(-expf(orc_bf16_to_float(a_log[h])) * gdn_softplus(a[h] + orc_bf16_to_float(dt_bias[h])));
        const float beta = 1.0f / (1.0f + expf(-b[h]));
        for (size_t d = 0; d < dv; ++d) {
            float *srow = state + (h * dv + d) * dk;
            float kv = 0.0f;
            for (size_t i = 0; i < dk; ++i) { srow[i] *= g; kv += srow[i] * k[i]; }
            const float delta = (v[d] - kv) * beta;
            float o = 0.0f;
            for (size_t i = 0; i < dk; ++i) { srow[i] += k[i] * delta; o += srow[i] * q[i]; }
            y[h * dv + d] = round_act(o, act);
        }
    }
    for (size_t h = 0; h < v_heads; ++h) {                    /* :102-112 */
        float sumsq = 0.0f;
        for (size_t i = 0; i < dv; ++i) sumsq += y[h * dv + i] * y[h * dv + i];
        const float inv = 1.0f / sqrtf(sumsq / (float)dv + 1e-6f);
        for (size_t i = 0; i < dv; ++i)
            out[h * dv + i] = y[h * dv + i] * inv * orc_bf16_to_float(norm_w[i]) * gdn_silu(z[h * dv + i]);
    }
    free(y); free(normed); free(conv);
}

/* Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293): for every DISTINCT id of the
 * history inside the vocabulary, a positive logit is divided by the penalty and a negative one
 * multiplied; with a logit softcap the penalty acts on the capped logit and is mapped back through
 * atanh.  logits are 16-bit activations held as floats; act 0 = bf16, 1 = fp16 (the reference). */
void orc_repetition_penalty(float *logits, int act, size_t v, const int32_t *ids, size_t n_ids,
                            float penalty, float softcap) {
    for (size_t j = 0; j < n_ids; ++j) {
        int seen = 0;                                          /* once per distinct id */
        for (size_t h = 0; h < j && !seen; ++h) seen = ids[h] == ids[j];
        if (seen || ids[j] < 0 || (size_t)ids[j] >= v) continue;
        const float z = logits[ids[j]];
        float out;
        if (softcap > 0.0f) {
            const float capped = softcap * tanhf(z / softcap);
            const float pen = capped > 0.0f ? capped / penalty : capped * penalty;
            const float limit = softcap * 0.9999f;
            const float clamped = fmaxf(fminf(pen, limit), -limit);
            out = softcap * atanhf(clamped / softcap);
        } else {
            out = z > 0.0f ? z / penalty : z * penalty;
        }
        logits[ids[j]] = act == 0 ? orc_bf16_to_float(orc_bf16_bits(out)) : orc_f16_to_float(orc_f16_bits(out));
    }
}

/* Sampler.sample's choice of kernel (Sampler.swift:196-231): 2 = the tiled top-64 sampler, 1 = the
 * generic kernel with its own three paths, 0 = generic greedy.  top_k <= 0 stands for nil. */
int orc_sampler_route(int tiled_path, float temperature, int top_k) {
    if (tiled_path && temperature > 0.0f && top_k >= 1 && top_k <= 64) return 2;
    return temperature == 0.0f ? 0 : 1;
}

/* Sampler.sample after the penalty: softcap + softmax, then the routed sampler with
 * seedFor(seed, position); top_p <= 0 stands for nil (1.0).  probs_f16 receives the probabilities. */
uint32_t orc_sampler_sample(const float *logits, size_t v, float softcap, int tiled_path,
                            float temperature, int top_k, float top_p, uint64_t seed,
                            int64_t position, uint16_t *probs_f16) {
    if (tiled_path) orc_softmax_tiled_f16(logits, v, softcap, probs_f16);
    else orc_softmax_f16(logits, v, softcap, probs_f16);
    const uint64_t s = orc_seed_for(seed, position);
    const float p = top_p > 0.0f ? top_p : 1.0f;
    if (orc_sampler_route(tiled_path, temperature, top_k) == 2)
        return orc_sample_topk64(probs_f16, v, temperature, p, s, (uint32_t)top_k, NULL, NULL);
    return orc_sample(probs_f16, v, temperature == 0.0f ? 0.0f : temperature,
                      top_k > 0 ? (uint32_t)top_k : 0u, p, s, (uint32_t)position);
}

float orc_rel_error(const float *actual, const float *reference, size_t n) {
    float max_diff = 0.0f, ref_norm = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        max_diff = fmaxf(max_diff, fabsf(actual[i] - reference[i]));
        ref_norm = fmaxf(ref_norm, fabsf(reference[i]));
    }
    return max_diff / fmaxf(ref_norm, 1e-6f);
}
