/* qk_oracle_mt.c -- the oracle's row loops spread over host threads.
 *
 * TEST INFRASTRUCTURE ONLY (see qk_oracle.c).  The reference's CPU path is single-threaded
 * (src/main.cpp:673-679, 1316-1387); the benchmark also wants that path on all host cores, rows split
 * across threads.  Every output element is computed by the same scalar code as in qk_oracle.c, by
 * exactly one thread, so the results are bit for bit those of the single-threaded functions
 * (tests/test_oracle.py pins that); nothing here is a second definition of the arithmetic.
 */
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "qk_oracle.h"

typedef void (*range_fn)(uint32_t lo, uint32_t hi, void *ctx);
typedef struct {
    range_fn fn;
    void *ctx;
    uint32_t lo, hi;
} range_job;

static void *run_range(void *p)
{
    range_job *j = (range_job *)p;
    j->fn(j->lo, j->hi, j->ctx);
    return NULL;
}

/* fn(lo, hi) over [0, n) cut into n_threads contiguous ranges; the calling thread takes the first. */
static void parallel_for(uint32_t n, uint32_t n_threads, range_fn fn, void *ctx)
{
    if (n_threads < 1) n_threads = 1;
    if (n_threads > n) n_threads = n ? n : 1;
    if (n_threads > 256) n_threads = 256;
    pthread_t th[256];
    range_job job[256];
    for (uint32_t t = 0; t < n_threads; t++) {
        job[t].fn = fn;
        job[t].ctx = ctx;
        job[t].lo = (uint32_t)((uint64_t)n * t / n_threads);
        job[t].hi = (uint32_t)((uint64_t)n * (t + 1) / n_threads);
    }
    for (uint32_t t = 1; t < n_threads; t++) pthread_create(&th[t], NULL, run_range, &job[t]);
    run_range(&job[0]);
    for (uint32_t t = 1; t < n_threads; t++) pthread_join(th[t], NULL);
}

/* ---- y[b][m] = W[m] . x[b], rows split (qko_gemv on each range) --------------------------- */
typedef struct {
    int type;
    const uint8_t *W;
    const float *x;
    float *y;
    uint32_t M, K, batch;
    size_t rb;
} gemv_ctx;

static void gemv_range(uint32_t lo, uint32_t hi, void *p)
{
    const gemv_ctx *c = (const gemv_ctx *)p;
    if (c->batch == 1) {
        qko_gemv(c->type, c->W + (size_t)lo * c->rb, c->x, c->y + lo, hi - lo, c->K, 1);
        return;
    }
    float *tmp = (float *)malloc((size_t)(hi - lo) * sizeof(float)); /* one activation row at a time: y's row stride is M */
    if (!tmp) return;
    for (uint32_t b = 0; b < c->batch; b++) {
        qko_gemv(c->type, c->W + (size_t)lo * c->rb, c->x + (size_t)b * c->K, tmp, hi - lo, c->K, 1);
        memcpy(c->y + (size_t)b * c->M + lo, tmp, (size_t)(hi - lo) * sizeof(float));
    }
    free(tmp);
}

int qko_gemv_mt(int type, const void *W, const float *x, float *y, uint32_t M, uint32_t K, uint32_t batch,
                uint32_t n_threads)
{
    gemv_ctx c = {type, (const uint8_t *)W, x, y, M, K, batch, qko_row_bytes(type, K)};
    if (c.rb == 0) return -1;
    parallel_for(M, n_threads, gemv_range, &c);
    return 0;
}

/* Y[n][m] = X[n] . dequant_q8_0(W[m]): the same split (a GEMM is the GEMV over N activation rows). */
int qko_gemm_q8_0_mt(const void *W, const float *X, float *Y, uint32_t M, uint32_t K, uint32_t N, uint32_t n_threads)
{
    return qko_gemv_mt(QKO_Q8_0, W, X, Y, M, K, N, n_threads);
}

/* ---- the fused MoE step of several tokens, tokens split (qko_moe_ref on each) ------------- */
typedef struct {
    const qko_moe_layer *L;
    const float *X;
    float *Y;
    int rc;
} moe_tok_ctx;

static void moe_tok_range(uint32_t lo, uint32_t hi, void *p)
{
    moe_tok_ctx *c = (moe_tok_ctx *)p;
    for (uint32_t t = lo; t < hi; t++)
        if (qko_moe_ref(c->L, c->X + (size_t)t * c->L->n_embd, c->Y + (size_t)t * c->L->n_embd, NULL, NULL, NULL)) c->rc = -1;
}

int qko_moe_ref_tokens_mt(const qko_moe_layer *L, const float *X, float *Y, uint32_t n_tokens, uint32_t n_threads)
{
    moe_tok_ctx c = {L, X, Y, 0};
    parallel_for(n_tokens, n_threads, moe_tok_range, &c);
    return c.rc;
}

/* ---- one token's step with its row loops split ------------------------------------------------
 * The steps of qko_moe_ref (src/main.cpp:1316-1387): router logits, selection, then per picked
 * expert (and the shared one) the gate/up rows and the down rows.  The logits come from the F32
 * GEMV and every expert row from the block GEMV (the same dequantise-then-double-dot), so y is
 * accumulated in the same order per element: routed picks in pick order, then the shared expert. */
typedef struct {
    int type;
    const uint8_t *g, *u;
    const float *x;
    float *h;
    uint32_t H;
    size_t rb;
} gu_ctx;

static void gu_range(uint32_t lo, uint32_t hi, void *p)
{
    const gu_ctx *c = (const gu_ctx *)p;
    float *row = (float *)malloc((size_t)c->H * sizeof(float));
    if (!row) return;
    for (uint32_t r = lo; r < hi; r++) {
        double ga = 0, ua = 0;
        qko_dequant_row(c->type, c->g + (size_t)r * c->rb, row, c->H);
        for (uint32_t i = 0; i < c->H; i++) ga += (double)row[i] * c->x[i];
        qko_dequant_row(c->type, c->u + (size_t)r * c->rb, row, c->H);
        for (uint32_t i = 0; i < c->H; i++) ua += (double)row[i] * c->x[i];
        c->h[r] = (float)((ga / (1.0 + exp(-ga))) * ua);
    }
    free(row);
}

typedef struct {
    int type;
    const uint8_t *d;
    const float *h;
    float *y;
    double wt;
    uint32_t F;
    size_t rb;
} dn_ctx;

static void dn_range(uint32_t lo, uint32_t hi, void *p)
{
    const dn_ctx *c = (const dn_ctx *)p;
    float *row = (float *)malloc((size_t)c->F * sizeof(float));
    if (!row) return;
    for (uint32_t o = lo; o < hi; o++) {
        double a = 0;
        qko_dequant_row(c->type, c->d + (size_t)o * c->rb, row, c->F);
        for (uint32_t i = 0; i < c->F; i++) a += (double)row[i] * c->h[i];
        c->y[o] += (float)(c->wt * a);
    }
    free(row);
}

typedef struct {
    const float *gi, *x;
    double *logit;
    uint32_t H;
} lg_ctx;

static void lg_range(uint32_t lo, uint32_t hi, void *p)
{
    const lg_ctx *c = (const lg_ctx *)p;
    for (uint32_t e = lo; e < hi; e++) {
        double a = 0;
        const float *r = c->gi + (size_t)e * c->H;
        for (uint32_t i = 0; i < c->H; i++) a += (double)r[i] * c->x[i];
        c->logit[e] = a;
    }
}

int qko_moe_ref_mt(const qko_moe_layer *L, const float *x, float *y, uint32_t n_threads)
{
    const uint32_t H = L->n_embd, F = L->n_ff, E = L->n_expert, k = L->n_used;
    const size_t rb_gu = qko_row_bytes(L->gu_type, H), rb_dn = qko_row_bytes(L->down_type, F);
    const size_t rb_sgu = qko_row_bytes(QKO_Q8_0, H), rb_sdn = qko_row_bytes(QKO_Q8_0, F);
    if (!rb_gu || !rb_dn || !rb_sgu || !rb_sdn || k < 1 || k > 16 || k > E) return -1;
    double *logit = (double *)malloc(E * sizeof(double));
    float *h = (float *)malloc(F * sizeof(float));
    if (!logit || !h) return -2;
    lg_ctx lc = {L->gate_inp, x, logit, H};
    parallel_for(E, n_threads, lg_range, &lc);
    qko_sel_f64 sel;
    qko_select_f64(logit, E, k, &sel);
    double sg = 0;
    for (uint32_t i = 0; i < H; i++) sg += (double)L->gate_inp_shexp[i] * x[i];
    sel.w_shared = 1.0 / (1.0 + exp(-sg));
    for (uint32_t o = 0; o < H; o++) y[o] = 0.f;
    for (uint32_t s = 0; s <= k; s++) {
        const int shared = s == k;
        gu_ctx gc = {shared ? QKO_Q8_0 : L->gu_type,
                     shared ? (const uint8_t *)L->gate_shexp : (const uint8_t *)L->gate_exps + (size_t)sel.ids[s] * F * rb_gu,
                     shared ? (const uint8_t *)L->up_shexp : (const uint8_t *)L->up_exps + (size_t)sel.ids[s] * F * rb_gu,
                     x, h, H, shared ? rb_sgu : rb_gu};
        parallel_for(F, n_threads, gu_range, &gc);
        dn_ctx dc = {shared ? QKO_Q8_0 : L->down_type,
                     shared ? (const uint8_t *)L->down_shexp : (const uint8_t *)L->down_exps + (size_t)sel.ids[s] * H * rb_dn,
                     h, y, shared ? sel.w_shared : sel.w[s], F, shared ? rb_sdn : rb_dn};
        parallel_for(H, n_threads, dn_range, &dc);
    }
    free(logit);
    free(h);
    return 0;
}
