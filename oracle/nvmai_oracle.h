/*
 * nvmai_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C CPU restatement of the reference's quantized mixture-of-experts
 * hot path (Pummelchen/NVMAI).  It exists only so that tests, the smoke check
 * and the bench's cpu_baseline leg can compare the HIP kernels against an
 * independent scalar implementation.  Nothing in the shipped library may link
 * or call it.
 *
 * Every function cites the reference file:line whose arithmetic it follows.
 * All float arithmetic is IEEE binary32, round-to-nearest-even; the file must
 * be compiled with -ffp-contract=off so that "a*b + c" is two roundings unless
 * fmaf() is written out.
 *
 * Pinning status (what fixes each function besides its own formula) is listed
 * at the top of nvmai_oracle.c.
 */
#ifndef NVMAI_ORACLE_H
#define NVMAI_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_GROUP 64

/* ---- scalar conversions ------------------------------------------------ */
uint16_t orc_bf16_bits(float x);           /* Quantization.swift:17-23 */
float orc_bf16_to_float(uint16_t bits);    /* Quantization.swift:26-28 */
uint16_t orc_f16_bits(float x);            /* IEEE binary16, RNE (Metal half(x)) */
float orc_f16_to_float(uint16_t bits);
void orc_round_through_bf16(float *v, size_t n);
void orc_round_through_f16(float *v, size_t n);

/* ---- test PRNGs -------------------------------------------------------- */
typedef struct { uint64_t state; } orc_splitmix64;
uint64_t orc_splitmix64_next(orc_splitmix64 *s);               /* SplitMix64.swift:11-17 */
float orc_splitmix64_uniform(orc_splitmix64 *s, float lo, float hi); /* :20-23 */
uint64_t orc_seedtree_key(uint64_t root, const char *label);   /* SeedTree.swift:12-19 */
/* CPUExpertFFNTests.swift:18-23: state = state*6364136223846793005 + inc */
float orc_lcg_next(uint64_t *state, uint64_t inc);

/* ---- affine group-64 weight quantizer ---------------------------------- */
/* Quantization.swift:50-102 (bits=4), :135-177 (bits=8).  rows x n, n%64==0.
 * packed: rows*n*bits/8 bytes, scales/biases: rows*(n/64) bf16 bit patterns. */
void orc_quantize_affine(const float *w, size_t rows, size_t n, int bits,
                         uint8_t *packed, uint16_t *scales, uint16_t *biases);
/* Quantization.swift:104-119, :179-191 */
void orc_dequantize_affine(const uint8_t *packed, const uint16_t *scales,
                           const uint16_t *biases, size_t rows, size_t n,
                           int bits, float *out);
/* codes only, one byte per element (the "unpacked codes" class) */
void orc_unpack_codes(const uint8_t *packed, size_t count, int bits, uint8_t *codes);

/* ---- expert blob layout (CPUExpertFFN.swift:42-59, MoE.swift:5-29) ------ */
/* out[0..8] = gate_W, gate_s, gate_b, up_W, up_s, up_b, down_W, down_s, down_b;
 * out[9] = stride bytes. */
void orc_expert_offsets(size_t d, size_t f, int bits, uint32_t out[10]);
/* Quantize gate[f,d], up[f,d], down[d,f] (fp32) into one blob. */
void orc_pack_expert(const float *gate, const float *up, const float *down,
                     size_t d, size_t f, int bits, uint8_t *blob);

/* ---- GEMV -------------------------------------------------------------- */
/* int4_affine_gemv.c:114-134 (portable path), same signature as the reference. */
void orc_int4_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                          const uint16_t *biases, const float *x, size_t rows,
                          size_t n, float *out);
/* Same factoring for bits in {4,8}: out[r] = sum_g s*dot_g + b*xsum_g
 * (dequant_int8.metal:67-107 states the 8-bit arithmetic). */
void orc_affine_gemv(const uint8_t *weights, const uint16_t *scales,
                     const uint16_t *biases, const float *x, size_t rows,
                     size_t n, int bits, float *out);
/* Unfactored: out[r] = sum_i (q*s+b)*x  (DequantInt4Gemv.swift:12-43). */
void orc_affine_gemv_unfactored(const uint8_t *weights, const uint16_t *scales,
                                const uint16_t *biases, const float *x,
                                size_t rows, size_t n, int bits, float *out);

/* ---- expert FFN (CPUExpertFFN.swift:101-139) ---------------------------- */
/* out[r] += route_w * down(silu(gate.x) * (up.x))[r]; scratch >= 2f+d floats */
void orc_expert_ffn_accumulate(const uint8_t *blob, const uint32_t off[10],
                               int bits, const float *x, size_t d, size_t f,
                               float route_w, float *scratch, float *out);

/* ---- router (moe.metal:174-285, prefill.metal:337-435) ------------------ */
/* Logits in the canonical lane order documented in nvmai_oracle.c.
 * kind: 8 or 4 = affine rows (weights/scales/biases), 16 = dense bf16 rows
 * (weights points at uint16 bf16 bits, scales/biases ignored).
 * eff_scale: optional bf16 bits [d] multiplied into x (NULL = 1.0). */
void orc_router_logits(const void *weights, const uint16_t *scales,
                       const uint16_t *biases, int kind, const float *x,
                       const uint16_t *eff_scale, size_t num_experts, size_t d,
                       float *logits);
/* moe.metal:233-285: top-k by (score desc, index asc); softmax over the
 * selected; times per-expert scale (bf16 bits, NULL = 1.0); weights as fp16 bits. */
void orc_router_topk(const float *logits, size_t num_experts, size_t k,
                     const uint16_t *per_expert_scale, uint32_t *out_idx,
                     uint16_t *out_w_f16);

/* One MoE layer for n_tokens independent tokens (RealForwardRunner.swift
 * :3866-3912 shared expert + :3914 routed; phase-2 residual = shared output).
 * experts: array of num_experts blob pointers; shared_blob may be NULL;
 * shared_gate_*: optional scalar gate row in router format (kind 0 = none).
 * y[t,:] = sigmoid(gate.x) * ffn_shared(x) + sum_slot w_slot * ffn_e(x). */
typedef struct {
    size_t d, f, num_experts, top_k;
    int bits;              /* expert weight bits */
    int router_kind;       /* 4, 8 or 16 */
    const void *router_w; const uint16_t *router_s; const uint16_t *router_b;
    const uint8_t *const *experts;
    const uint8_t *shared_blob;
    int gate_kind;         /* 0 none, else 4/8/16 */
    const void *gate_w; const uint16_t *gate_s; const uint16_t *gate_b;
} orc_moe_layer;
void orc_moe_layer_forward(const orc_moe_layer *L, const float *x, size_t n_tokens,
                           uint32_t *out_idx, uint16_t *out_w_f16, float *y);

/* ---- prefill grouping (PrefillRouter.swift:97-117, PrefillMoEGrouping.swift) */
typedef struct { uint32_t token, expert, rank, weight_bits; } orc_pair;
typedef struct { uint32_t expert, pair_start, pair_count; } orc_group;
typedef struct { uint32_t group_start, group_count, pair_start, pair_count; } orc_tile;
void orc_make_pairs(const uint32_t *idx, const uint16_t *w_f16, size_t tokens,
                    size_t k, orc_pair *pairs);
/* error codes mirror PrefillMoEGroupingError */
enum {
    ORC_GROUP_OK = 0, ORC_GROUP_BAD_QUERY = -1, ORC_GROUP_BAD_TOPK = -2,
    ORC_GROUP_BAD_EXPERTS = -3, ORC_GROUP_BAD_TILE = -4, ORC_GROUP_PAIR_COUNT = -5,
    ORC_GROUP_TOKEN_RANGE = -6, ORC_GROUP_RANK_RANGE = -7, ORC_GROUP_EXPERT_RANGE = -8,
    ORC_GROUP_DUPLICATE = -9, ORC_GROUP_SORTKEY_COUNT = -10
};
/* sorted: n_pairs; offsets/counts: num_experts; groups: up to num_experts;
 * tiles: up to num_experts.  sort_keys may be NULL (n_sort_keys ignored then). */
int orc_group_pairs(const orc_pair *pairs, size_t n_pairs, long query_count,
                    long top_k, long num_experts, long tile_expert_count,
                    const uint64_t *sort_keys, size_t n_sort_keys,
                    orc_pair *sorted, uint32_t *offsets, uint32_t *counts,
                    orc_group *groups, size_t *n_groups, orc_tile *tiles,
                    size_t *n_tiles);
/* Routed prefill MoE: h2[t,:] = sum_r fma(w[t,r], ffn_{e(t,r)}(x_t), acc)
 * (prefill.metal:437-534 with fp32 intermediates as on the CPU path). */
void orc_prefill_moe(const uint8_t *const *experts, const uint32_t off[10],
                     int bits, const float *x, size_t tokens, size_t d, size_t f,
                     size_t k, const uint32_t *idx, const uint16_t *w_f16, float *h2);

/* ---- KV cache ---------------------------------------------------------- */
/* KVCacheManager.swift:437-446 */
void orc_kv_row_layout(size_t elements, int bits, size_t *stride, size_t *value_bytes);
/* kv_cache_quantize.metal:7-73; src[token*src_stride + i] already holds the
 * activation-dtype values as float. */
void orc_kv_quantize(const float *src, size_t src_stride, size_t tokens,
                     size_t elements, int bits, uint8_t *dst, size_t dst_stride,
                     size_t value_bytes);
/* attention.metal:89-117 */
void orc_kv_dequant_row(const uint8_t *row, size_t elements, int bits,
                        size_t value_bytes, float *out);
/* rope.metal:32-50,80-102: in-place on data[tokens, heads, head_dim] */
void orc_rope_neox_subdim(float *data, size_t tokens, size_t heads, size_t head_dim,
                          size_t rotary_dim, const uint32_t *positions, float theta);
/* Attention.swift:142-168 */
void orc_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len,
                        uint32_t kv_start, int prefer_gqa_swa, uint32_t *eff_len,
                        uint32_t *num_chunks, uint32_t *chunk_len,
                        uint32_t *partial_groups);
/* Decode attention for one sequence.  K/V rows: bits 4/8 = quantized rows of
 * `stride` bytes, bits 32 = float rows of elements floats.  num_chunks==0 ->
 * single pass (AttentionRef, Attention.swift:9-108 of the validation support);
 * else split-KV with the given chunk_len (attention.metal:163-261,388-429).
 * out: [num_q_heads, head_dim] float (not rounded). */
void orc_attention_decode(const float *q, const void *k, const void *v, int kv_bits,
                          size_t stride, size_t value_bytes, size_t num_q_heads,
                          size_t num_kv_heads, size_t head_dim, size_t seq_len,
                          size_t kv_start, float scale, size_t num_chunks,
                          size_t chunk_len, float *out);

/* Causal prefill attention, attention_prefill_causal_tiled (prefill.metal:709-830): query t
 * (row q + t * q_stride, [num_q_heads, head_dim]) at absolute position start + t attends to
 * keys [first, min(kv_valid, start + t + 1)) with first = start + t + 1 - window when window
 * != 0 and that is positive, else 0 (:760-764); online softmax over the keys in ascending
 * order (:771-792), out = acc / row_sum, zeros for an empty row (:794-797).  The row of key p
 * is p % ring when ring != 0 (:732-737).  K/V rows as for orc_attention_decode.  out row t at
 * out + t * out_stride, not rounded. */
void orc_attention_prefill_causal(const float *q, size_t q_stride, const void *k, const void *v,
                                  int kv_bits, size_t stride, size_t value_bytes,
                                  size_t num_q_heads, size_t num_kv_heads, size_t head_dim,
                                  size_t start, size_t count, size_t kv_valid, size_t window,
                                  size_t ring, float scale, float *out, size_t out_stride);

/* ---- softmax + sampler (logit.metal) ------------------------------------ */
/* two-pass fp32 softmax with optional softcap (<=0 disables), fp16 probs */
void orc_softmax_f16(const float *logits, size_t v, float softcap, uint16_t *probs_f16);
/* tiled online form, logit.metal:152-257 with tile 4096 */
void orc_softmax_tiled_f16(const float *logits, size_t v, float softcap,
                           uint16_t *probs_f16);
uint64_t orc_xorshift64star(uint64_t *s);            /* logit.metal:280-285 */
float orc_uniform01(uint64_t *s);                    /* logit.metal:287-292 */
uint64_t orc_seed_for(uint64_t seed, int64_t position); /* Sampler.swift:304-325 */
/* generic `sample` (logit.metal:315-585): k argmax passes */
/* Gumbel-max path (logit.metal:296-313, 391-429) and the kernel's choice of path. */
float orc_gumbel_for(uint64_t seed, uint32_t position, uint32_t row);
uint32_t orc_sample_gumbel(const uint16_t *probs_f16, size_t v, float temperature,
                           uint64_t seed, uint32_t position);
uint32_t orc_sample(const uint16_t *probs_f16, size_t v, float temperature, uint32_t top_k,
                    float top_p, uint64_t seed, uint32_t position);
uint32_t orc_sample_generic(const uint16_t *probs_f16, size_t v, float temperature,
                            uint32_t top_k, float top_p, uint64_t seed);
/* tiled top-64 (logit.metal:590-758): returns token; if top64_idx/val non-NULL
 * also returns the final 64 candidates */
uint32_t orc_sample_topk64(const uint16_t *probs_f16, size_t v, float temperature,
                           float top_p, uint64_t seed, uint32_t top_k,
                           uint32_t *top64_idx, float *top64_val);

/* GDNReference.step (GDNReference.swift:41-114): one token of gated-DeltaNet linear attention --
 * causal depthwise conv + SiLU, q / k norm with folded scales, gated delta rule, gated output norm. */
void orc_gdn_step(const float *qkv_raw, const float *a, const float *b, const float *z,
                  const uint16_t *conv_w, const uint16_t *a_log, const uint16_t *dt_bias,
                  const uint16_t *norm_w, size_t k_heads, size_t v_heads, size_t dk, size_t dv,
                  size_t taps, int act, float *tail, float *state, float *out);

/* Sampler.sample's front end (Sampler.swift:171-293): the repetition penalty over the distinct
 * history ids, the choice between the tiled and the generic sampler, and the whole call. */
void orc_repetition_penalty(float *logits, int act, size_t v, const int32_t *ids, size_t n_ids,
                            float penalty, float softcap);
int orc_sampler_route(int tiled_path, float temperature, int top_k);
uint32_t orc_sampler_sample(const float *logits, size_t v, float softcap, int tiled_path,
                            float temperature, int top_k, float top_p, uint64_t seed,
                            int64_t position, uint16_t *probs_f16);

/* RelError.swift:5-16 */
/* ---- rest of the decode step ------------------------------------------- */
void orc_rmsnorm(const float *x, size_t x_stride, const uint16_t *weight_bf16, size_t rows,
                 size_t d, float eps, float *out, size_t out_stride);   /* rmsnorm.metal:31-170 */
void orc_elementwise(int op, const float *a, const float *b, size_t count, float *out); /* utility.metal:32-104 */
void orc_embed_lookup(const uint8_t *table, const uint16_t *scales, const uint16_t *biases,
                      int bits, uint32_t token, size_t vocab, size_t d, float out_scale,
                      float *out);                                      /* dequant_int4.metal:63-91 */
uint32_t orc_lm_head_greedy(const float *hidden, const uint16_t *norm_weight_bf16,
                            const uint8_t *weights, const uint16_t *scales,
                            const uint16_t *biases, int bits, size_t d, size_t vocab,
                            float eps, int act, float *logits_out);     /* logit.metal:761-937 */

float orc_rel_error(const float *actual, const float *reference, size_t n);

#ifdef __cplusplus
}
#endif
#endif
