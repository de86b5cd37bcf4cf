/*
 * nvmai_oracle_bench.c -- timing loops around the CPU oracle: TEST / BENCH INFRASTRUCTURE, not
 * product code.  Only bench.py's cpu_baseline leg calls it.
 *
 * The reference's CPU path has no threads of its own; its published multi-thread numbers
 * partition independent work over threads (docs/cpu-coexecution-plan.md:45-50).  Here each
 * thread takes a static share of the independent units (tokens of a decode step, pairs of a
 * prefill block, query-head groups of an attention call).  Timing: CLOCK_MONOTONIC around each
 * repetition after `warmup` untimed ones; the median is returned.
 */
#define _POSIX_C_SOURCE 200809L
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "nvmai_oracle.h"

static double now_s(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

static int cmp_double(const void *a, const void *b) {
    const double x = *(const double *)a, y = *(const double *)b;
    return x < y ? -1 : x > y;
}

typedef void (*unit_fn)(void *job, size_t first, size_t count);
typedef struct { unit_fn fn; void *job; size_t first, count; } share;

static void *run_share(void *p) {
    share *s = (share *)p;
    if (s->count) s->fn(s->job, s->first, s->count);
    return NULL;
}

/* units 0..n-1 in contiguous shares over `threads` threads; returns the median wall time */
static double time_shares(unit_fn fn, void *job, size_t n, int threads, int warmup, int reps) {
    if (threads < 1) threads = 1;
    if ((size_t)threads > n) threads = (int)n;
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    share *sh = (share *)malloc(sizeof(share) * (size_t)threads);
    double *t = (double *)malloc(sizeof(double) * (size_t)(reps > 0 ? reps : 1));
    for (int r = -warmup; r < reps; ++r) {
        const double t0 = now_s();
        size_t at = 0;
        for (int i = 0; i < threads; ++i) {
            const size_t cnt = n / (size_t)threads + ((size_t)i < n % (size_t)threads ? 1 : 0);
            sh[i].fn = fn; sh[i].job = job; sh[i].first = at; sh[i].count = cnt;
            at += cnt;
            if (i > 0) pthread_create(&tid[i], NULL, run_share, &sh[i]);
        }
        run_share(&sh[0]);
        for (int i = 1; i < threads; ++i) pthread_join(tid[i], NULL);
        if (r >= 0) t[r] = now_s() - t0;
    }
    qsort(t, (size_t)reps, sizeof(double), cmp_double);
    const double med = t[reps / 2];
    free(t); free(sh); free(tid);
    return med;
}

/* ---- configs[1]: MoE-layer decode step, tokens shared out ---------------------------------- */
typedef struct { const orc_moe_layer *L; const float *x; uint32_t *idx; uint16_t *w; float *y; } moe_job;
static void moe_unit(void *job, size_t first, size_t count) {
    moe_job *j = (moe_job *)job;
    orc_moe_layer_forward(j->L, j->x + first * j->L->d, count, j->idx + first * j->L->top_k,
                          j->w + first * j->L->top_k, j->y + first * j->L->d);
}
double orc_time_moe_layer(const orc_moe_layer *L, const float *x, size_t n_tokens, int threads,
                          int warmup, int reps, uint32_t *out_idx, uint16_t *out_w, float *y) {
    moe_job j = {L, x, out_idx, out_w, y};
    return time_shares(moe_unit, &j, n_tokens, threads, warmup, reps);
}

/* ---- configs[3]: decode attention, sequences shared out ------------------------------------- */
typedef struct {
    const float *q; const uint8_t *k, *v; size_t kv_seq_stride; int bits; size_t stride, value_bytes, nq, nkv, hd, seq;
    float scale; float *out;
} attn_job;
static void attn_unit(void *job, size_t first, size_t count) {
    attn_job *j = (attn_job *)job;
    for (size_t b = first; b < first + count; ++b)
        orc_attention_decode(j->q + b * j->nq * j->hd, j->k + b * j->kv_seq_stride, j->v + b * j->kv_seq_stride,
                             j->bits, j->stride, j->value_bytes, j->nq, j->nkv, j->hd, j->seq, 0, j->scale, 0, 0,
                             j->out + b * j->nq * j->hd);
}
/* q, out: [sequences, nq, hd]; k, v: sequence b's rows at k + b * kv_seq_stride bytes */
double orc_time_attention(const float *q, const uint8_t *k, const uint8_t *v, size_t kv_seq_stride,
                          size_t sequences, int bits, size_t stride, size_t value_bytes, size_t nq,
                          size_t nkv, size_t hd, size_t seq, float scale, int threads, int warmup,
                          int reps, float *out) {
    attn_job j = {q, k, v, kv_seq_stride, bits, stride, value_bytes, nq, nkv, hd, seq, scale, out};
    return time_shares(attn_unit, &j, sequences, threads, warmup, reps);
}

/* ---- configs[2]: prefill MoE over a few tokens, tokens shared out --------------------------- */
typedef struct {
    const uint8_t *const *experts; const uint32_t *off; int bits; const float *x; size_t d, f, k;
    const uint32_t *idx; const uint16_t *w; float *h2;
} pf_job;
static void pf_unit(void *job, size_t first, size_t count) {
    pf_job *j = (pf_job *)job;
    orc_prefill_moe(j->experts, j->off, j->bits, j->x + first * j->d, count, j->d, j->f, j->k,
                    j->idx + first * j->k, j->w + first * j->k, j->h2 + first * j->d);
}
double orc_time_prefill_moe(const uint8_t *const *experts, const uint32_t *off, int bits, const float *x,
                            size_t tokens, size_t d, size_t f, size_t k, const uint32_t *idx,
                            const uint16_t *w, int threads, int warmup, int reps, float *h2) {
    pf_job j = {experts, off, bits, x, d, f, k, idx, w, h2};
    return time_shares(pf_unit, &j, tokens, threads, warmup, reps);
}
