/* qk_oracle.c -- CPU oracle for the quantized-weight decode hot path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by tests/, by the smoke check and by the
 * cpu_baseline leg of the benchmark; the product library never calls it.
 *
 * It restates, in scalar C, what the reference computes on the CPU for this
 * path (paths relative to /root/reference):
 *   half conversions, block layouts, dequantisation ... src/quants.h
 *   codebooks ........................................ src/quant_tables.h
 *   row dot product in double ........................ src/main.cpp:626-633, 673-679
 *   fused MoE step ................................... src/main.cpp:1316-1387
 *   greedy argmax .................................... src/main.cpp:5387-5388
 *   selector tie / non-finite rules .................. shaders/moe_select.comp
 *   pair grouping .................................... shaders/moe_group_pairs.comp
 *   batched GEMM reference and acceptance ............ src/main.cpp:5561-5570, 5653-5662
 *   scale-aware acceptance metric .................... src/main.cpp:548-565
 *   RMS norm (with the shaders' fp32 residual sums) .. src/main.cpp:1685-1690, shaders/add_rms3.comp:29-40
 *   embedding lookup ................................. shaders/embed_q6k.comp:27-49
 *
 * How each part is pinned (tests/test_oracle.py, tests/test_golden.py):
 *   qko_f16_to_f32 / qko_f32_to_f16 .. all 65,536 halves and a float sweep against the
 *       reference build (oracle/_ref) and against the compiler's _Float16 where the
 *       reference agrees with IEEE (it flushes results below 2^-14 to zero).
 *   qko_dequant_row (4 formats) ....... bitwise against oracle/_ref on seeded random
 *       blocks and against the committed vectors in tests/golden/, plus closed forms
 *       (all-zero fields, single-codeword blocks).
 *   qko_ksign ......................... all 128 entries against the reference table.
 *   qko_gemv / qko_gemm_q8_0 .......... against numpy float64 matmul on the dequantised rows.
 *   qko_select_f64 / qko_select_f32 ... against numpy argsort and softmax; invariants
 *       (weights sum to 1, descending, ids distinct); tie and NaN cases.
 *   qko_moe_ref ....................... against a dense numpy float64 evaluation that
 *       dequantises every expert; the k = n_expert special case equals a dense
 *       softmax-weighted MLP.
 *   qko_group_pairs ................... against a numpy stable sort.
 *   qko_argmax ........................ against numpy argmax, with duplicated maxima.
 *   qko_add_rms ....................... against a numpy float64 evaluation; unit weights give
 *       mean(xn^2) = ms/(ms+eps); scaling the inputs by 2 leaves xn unchanged at eps = 0
 *       (exact in binary floating point); the stored sum is bitwise numpy's float32 (a+b)+c.
 *   qko_embed ......................... bitwise qko_dequant_row of the chosen rows.
 * Agreement of these formats with upstream ggml is pinned in the reference only by
 * model-level token parity, which needs a model file that is absent here: parity
 * with upstream ggml is unpinned; parity with the reference's header is pinned.
 */
#include "qk_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "qk_oracle_tables.h"

/* ---- half <-> float (src/quants.h:12-48) --------------------------------- */

float qko_f16_to_f32(uint16_t h)
{
    const uint32_t s = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 31u) {
        bits = s | 0x7F800000u | (m << 13); /* Inf / NaN keep their payload */
    } else if (e != 0u) {
        bits = s | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        bits = s;
    } else { /* subnormal half: normalise */
        e = 113u;
        do {
            m <<= 1;
            e--;
        } while ((m & 1024u) == 0u);
        bits = s | (e << 23) | ((m & 1023u) << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

uint16_t qko_f32_to_f16(float f)
{
    uint32_t bits;
    memcpy(&bits, &f, sizeof bits);
    const uint32_t s = (bits >> 16) & 0x8000u;
    const int32_t e = (int32_t)((bits >> 23) & 255u) - 112;
    const uint32_t m = bits & 0x7FFFFFu;
    if (e <= 0) return (uint16_t)s;             /* the reference flushes anything below 2^-14 */
    if (e >= 31) return (uint16_t)(s | 0x7C00u); /* overflow, Inf and NaN all become Inf */
    uint32_t h = s | ((uint32_t)e << 10) | (m >> 13);
    const uint32_t tail = m & 0x1FFFu;
    if (tail > 0x1000u || (tail == 0x1000u && (h & 1u))) h++; /* nearest even; may carry into exp */
    return (uint16_t)h;
}

uint8_t qko_ksign(uint32_t i)
{
    i &= 127u;
    uint32_t p = i;
    p ^= p >> 4;
    p ^= p >> 2;
    p ^= p >> 1;
    return (uint8_t)(i | ((p & 1u) << 7));
}

/* ---- block geometry (src/quants.h:51-66, 107-119; src/gguf.h:36-46) ------- */

enum { Q8_0_BYTES = 34, Q6_K_BYTES = 210, IQ4_XS_BYTES = 136, IQ3_XXS_BYTES = 98 };

size_t qko_row_bytes(int type, uint64_t k)
{
    switch (type) {
    case QKO_F32: return (size_t)k * 4;
    case QKO_F16: return (size_t)k * 2;
    case QKO_Q8_0: return k % 32 ? 0 : (size_t)(k / 32) * Q8_0_BYTES;
    case QKO_Q6_K: return k % 256 ? 0 : (size_t)(k / 256) * Q6_K_BYTES;
    case QKO_IQ4_XS: return k % 256 ? 0 : (size_t)(k / 256) * IQ4_XS_BYTES;
    case QKO_IQ3_XXS: return k % 256 ? 0 : (size_t)(k / 256) * IQ3_XXS_BYTES;
    default: return 0;
    }
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static uint32_t rd32(const uint8_t *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* Q8_0: {f16 d; int8 q[32]}; w = d*q  (src/quants.h:70-77). */
static void dq_q8_0(const uint8_t *b, float *y)
{
    const float d = qko_f16_to_f32(rd16(b));
    for (int j = 0; j < 32; j++) y[j] = d * (float)(int8_t)b[2 + j];
}

/* Q6_K: {u8 ql[128]; u8 qh[64]; i8 sc[16]; f16 d}; element e of the block:
 * half n=e/128, quarter c=(e%128)/32, l=e%32; low nibble source ql[64n + 32(c&1) + l],
 * taken high when c>=2; two high bits from qh[32n + l] >> 2c; scale sc[8n + 2c + l/16];
 * w = d*sc*(q-32), evaluated left to right (src/quants.h:79-105). */
static void dq_q6_K(const uint8_t *b, float *y)
{
    const uint8_t *ql = b, *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    const float d = qko_f16_to_f32(rd16(b + 208));
    for (int e = 0; e < 256; e++) {
        const int n = e >> 7, c = (e >> 5) & 3, l = e & 31;
        const uint8_t lo = ql[64 * n + 32 * (c & 1) + l];
        const int nib = c >= 2 ? lo >> 4 : lo & 15;
        const int hi2 = (qh[32 * n + l] >> (2 * c)) & 3;
        const int8_t q = (int8_t)((int8_t)(nib | (hi2 << 4)) - 32);
        y[e] = d * (float)sc[8 * n + 2 * c + l / 16] * (float)q;
    }
}

/* IQ4_XS: {f16 d; u16 scales_h; u8 scales_l[4]; u8 qs[128]}; sub-block ib of 32:
 * ls = 4 low bits from scales_l, 2 high bits from scales_h; dl = d*(ls-32);
 * qs byte j of the sub-block feeds element j (low nibble) and j+16 (high)
 * (src/quants.h:121-139). */
static void dq_iq4_xs(const uint8_t *b, float *y)
{
    const float d = qko_f16_to_f32(rd16(b));
    const uint32_t sh = rd16(b + 2);
    for (int ib = 0; ib < 8; ib++) {
        const int lo4 = (b[4 + ib / 2] >> (4 * (ib & 1))) & 15;
        const int hi2 = (int)((sh >> (2 * ib)) & 3u);
        const float dl = d * (float)((lo4 | (hi2 << 4)) - 32);
        const uint8_t *q = b + 8 + 16 * ib;
        for (int j = 0; j < 16; j++) {
            y[32 * ib + j] = dl * (float)qko_iq4nl_values[q[j] & 15];
            y[32 * ib + 16 + j] = dl * (float)qko_iq4nl_values[q[j] >> 4];
        }
    }
}

/* IQ3_XXS: {f16 d; u8 qs[64]; u32 aux[8]}; group ib of 32 elements: aux packs four
 * 7-bit sign selectors and a 4-bit scale; db = d*(0.5+scale)*0.5; each 8 elements take
 * two grid codewords (4 magnitudes each) and one sign byte (src/quants.h:141-165). */
static void dq_iq3_xxs(const uint8_t *b, float *y)
{
    const float d = qko_f16_to_f32(rd16(b));
    for (int ib = 0; ib < 8; ib++) {
        const uint32_t aux = rd32(b + 2 + 64 + 4 * ib);
        const float db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
        for (int l = 0; l < 4; l++) {
            const uint8_t sg = qko_ksign((aux >> (7 * l)) & 127u);
            for (int half = 0; half < 2; half++) {
                const uint32_t cw = qko_iq3xxs_grid[b[2 + 8 * ib + 2 * l + half]];
                for (int j = 0; j < 4; j++) {
                    const float mag = (float)((cw >> (8 * j)) & 255u);
                    const float sgn = (sg >> (4 * half + j)) & 1 ? -1.f : 1.f;
                    y[32 * ib + 8 * l + 4 * half + j] = db * mag * sgn;
                }
            }
        }
    }
}

int qko_dequant_row(int type, const void *row, float *y, int64_t k)
{
    const uint8_t *p = (const uint8_t *)row;
    if (k < 0 || (k > 0 && qko_row_bytes(type, (uint64_t)k) == 0)) return -1;
    switch (type) {
    case QKO_F32: memcpy(y, p, (size_t)k * 4); return 0;
    case QKO_F16:
        for (int64_t i = 0; i < k; i++) y[i] = qko_f16_to_f32(rd16(p + 2 * i));
        return 0;
    case QKO_Q8_0:
        for (int64_t i = 0; i < k / 32; i++) dq_q8_0(p + i * Q8_0_BYTES, y + 32 * i);
        return 0;
    case QKO_Q6_K:
        for (int64_t i = 0; i < k / 256; i++) dq_q6_K(p + i * Q6_K_BYTES, y + 256 * i);
        return 0;
    case QKO_IQ4_XS:
        for (int64_t i = 0; i < k / 256; i++) dq_iq4_xs(p + i * IQ4_XS_BYTES, y + 256 * i);
        return 0;
    case QKO_IQ3_XXS:
        for (int64_t i = 0; i < k / 256; i++) dq_iq3_xxs(p + i * IQ3_XXS_BYTES, y + 256 * i);
        return 0;
    default: return -1;
    }
}

/* ---- dot products --------------------------------------------------------- */

static double dot_f64(const float *a, const float *b, uint32_t n)
{
    double acc = 0;
    for (uint32_t i = 0; i < n; i++) acc += (double)a[i] * b[i];
    return acc;
}

int qko_gemv(int type, const void *W, const float *x, float *y, uint32_t M, uint32_t K,
             uint32_t batch)
{
    const size_t rb = qko_row_bytes(type, K);
    if (rb == 0) return -1;
    float *tmp = (float *)malloc((size_t)K * sizeof(float));
    if (!tmp) return -2;
    for (uint32_t m = 0; m < M; m++) {
        qko_dequant_row(type, (const uint8_t *)W + (size_t)m * rb, tmp, K);
        for (uint32_t b = 0; b < batch; b++)
            y[(size_t)b * M + m] = (float)dot_f64(tmp, x + (size_t)b * K, K);
    }
    free(tmp);
    return 0;
}

int qko_gemm_q8_0(const void *W, const float *X, float *Y, uint32_t M, uint32_t K, uint32_t N)
{
    const size_t rb = qko_row_bytes(QKO_Q8_0, K);
    if (rb == 0) return -1;
    float *tmp = (float *)malloc((size_t)K * sizeof(float));
    if (!tmp) return -2;
    for (uint32_t m = 0; m < M; m++) {
        qko_dequant_row(QKO_Q8_0, (const uint8_t *)W + (size_t)m * rb, tmp, K);
        for (uint32_t n = 0; n < N; n++)
            Y[(size_t)n * M + m] = (float)dot_f64(tmp, X + (size_t)n * K, K);
    }
    free(tmp);
    return 0;
}

uint32_t qko_argmax(const float *v, uint32_t n)
{
    uint32_t best = 0;
    for (uint32_t i = 1; i < n; i++)
        if (v[i] > v[best]) best = i;
    return best;
}

/* ---- router ---------------------------------------------------------------- */

void qko_select_f64(const double *logits, uint32_t n_expert, uint32_t n_used, qko_sel_f64 *out)
{
    uint8_t *taken = (uint8_t *)calloc(n_expert, 1);
    memset(out, 0, sizeof *out);
    for (uint32_t i = 0; i < n_used; i++) {
        uint32_t best = n_expert;
        for (uint32_t e = 0; e < n_expert; e++) {
            if (taken[e]) continue;
            if (best == n_expert || logits[e] > logits[best]) best = e;
        }
        taken[best] = 1;
        out->ids[i] = best;
    }
    const double top = logits[out->ids[0]];
    double sum = 0;
    for (uint32_t i = 0; i < n_used; i++) {
        out->w[i] = exp(logits[out->ids[i]] - top);
        sum += out->w[i];
    }
    for (uint32_t i = 0; i < n_used; i++) out->w[i] /= sum;
    double runner = -INFINITY;
    for (uint32_t e = 0; e < n_expert; e++)
        if (!taken[e] && logits[e] > runner) runner = logits[e];
    out->gap = logits[out->ids[n_used - 1]] - runner;
    free(taken);
}

void qko_select_f32(const float *logits, uint32_t n_expert, uint32_t n_used, qko_sel *out)
{
    const float floor_v = -3.4e38f;
    float *l = (float *)malloc(n_expert * sizeof(float));
    memset(out, 0, sizeof *out);
    for (uint32_t e = 0; e < n_expert; e++)
        l[e] = (isnan(logits[e]) || isinf(logits[e])) ? floor_v : logits[e];
    float picked[16];
    for (uint32_t i = 0; i < n_used; i++) {
        uint32_t best = 0;
        for (uint32_t e = 1; e < n_expert; e++)
            if (l[e] > l[best]) best = e;
        out->ids[i] = best < n_expert ? best : n_expert - 1;
        picked[i] = l[best];
        l[best] = floor_v;
    }
    float sum = 0.f;
    for (uint32_t i = 0; i < n_used; i++) {
        out->w[i] = expf(picked[i] - picked[0]);
        sum += out->w[i];
    }
    for (uint32_t i = 0; i < n_used; i++) out->w[i] /= sum;
    free(l);
}

/* ---- fused MoE step (src/main.cpp:1316-1387) -------------------------------- */

static double silu_f64(double v) { return v / (1.0 + exp(-v)); }

int qko_moe_ref(const qko_moe_layer *L, const float *x, float *y, qko_sel_f64 *sel_out, float *h_out,
                double *logits_out)
{
    const uint32_t H = L->n_embd, F = L->n_ff, E = L->n_expert, k = L->n_used;
    const size_t rb_gu = qko_row_bytes(L->gu_type, H);
    const size_t rb_dn = qko_row_bytes(L->down_type, F);
    const size_t rb_sgu = qko_row_bytes(QKO_Q8_0, H);
    const size_t rb_sdn = qko_row_bytes(QKO_Q8_0, F);
    if (!rb_gu || !rb_dn || !rb_sgu || !rb_sdn || k < 1 || k > 16 || k > E) return -1;

    double *logit = (double *)malloc(E * sizeof(double));
    float *rowH = (float *)malloc(H * sizeof(float));
    float *rowF = (float *)malloc(F * sizeof(float));
    float *hrow = (float *)malloc(F * sizeof(float));
    if (!logit || !rowH || !rowF || !hrow) return -2;

    for (uint32_t e = 0; e < E; e++) logit[e] = dot_f64(L->gate_inp + (size_t)e * H, x, H);
    qko_sel_f64 sel;
    qko_select_f64(logit, E, k, &sel);
    sel.w_shared = 1.0 / (1.0 + exp(-dot_f64(L->gate_inp_shexp, x, H)));

    for (uint32_t o = 0; o < H; o++) y[o] = 0.f;
    for (uint32_t s = 0; s <= k; s++) { /* s == k is the shared expert */
        const int shared = s == k;
        const uint8_t *g = shared ? (const uint8_t *)L->gate_shexp
                                  : (const uint8_t *)L->gate_exps + (size_t)sel.ids[s] * F * rb_gu;
        const uint8_t *u = shared ? (const uint8_t *)L->up_shexp
                                  : (const uint8_t *)L->up_exps + (size_t)sel.ids[s] * F * rb_gu;
        const uint8_t *dn = shared ? (const uint8_t *)L->down_shexp
                                   : (const uint8_t *)L->down_exps + (size_t)sel.ids[s] * H * rb_dn;
        const int t_gu = shared ? QKO_Q8_0 : L->gu_type;
        const int t_dn = shared ? QKO_Q8_0 : L->down_type;
        const size_t b_gu = shared ? rb_sgu : rb_gu, b_dn = shared ? rb_sdn : rb_dn;
        const double wt = shared ? sel.w_shared : sel.w[s];
        for (uint32_t r = 0; r < F; r++) {
            qko_dequant_row(t_gu, g + (size_t)r * b_gu, rowH, H);
            const double ga = dot_f64(rowH, x, H);
            qko_dequant_row(t_gu, u + (size_t)r * b_gu, rowH, H);
            const double ua = dot_f64(rowH, x, H);
            hrow[r] = (float)(silu_f64(ga) * ua);
        }
        if (h_out) memcpy(h_out + (size_t)s * F, hrow, F * sizeof(float));
        for (uint32_t o = 0; o < H; o++) {
            qko_dequant_row(t_dn, dn + (size_t)o * b_dn, rowF, F);
            y[o] += (float)(wt * dot_f64(rowF, hrow, F));
        }
    }
    if (sel_out) *sel_out = sel;
    if (logits_out) memcpy(logits_out, logit, E * sizeof(double));
    free(logit);
    free(rowH);
    free(rowF);
    free(hrow);
    return 0;
}

/* ---- pair grouping (shaders/moe_group_pairs.comp:19-51) --------------------- */

int qko_group_pairs(const qko_sel *sel, uint32_t n_tokens, uint32_t n_expert, uint32_t n_used,
                    uint32_t *offsets, uint32_t *pairs)
{
    if (n_used < 1 || n_used > 16 || n_expert < 1) return -1;
    uint32_t *cursor = (uint32_t *)calloc(n_expert + 1, sizeof(uint32_t));
    if (!cursor) return -2;
    const uint32_t np = n_tokens * n_used;
    for (uint32_t p = 0; p < np; p++) {
        uint32_t e = sel[p / n_used].ids[p % n_used];
        if (e > n_expert - 1) e = n_expert - 1;
        cursor[e + 1]++;
    }
    for (uint32_t e = 0; e < n_expert; e++) cursor[e + 1] += cursor[e];
    memcpy(offsets, cursor, (n_expert + 1) * sizeof(uint32_t));
    for (uint32_t p = 0; p < np; p++) {
        const uint32_t t = p / n_used, s = p % n_used;
        uint32_t e = sel[t].ids[s];
        if (e > n_expert - 1) e = n_expert - 1;
        pairs[cursor[e]++] = (t << 4) | s;
    }
    free(cursor);
    return 0;
}

/* ---- acceptance metrics ----------------------------------------------------- */

static double rms_of(const float *v, size_t n)
{
    double s = 0;
    for (size_t i = 0; i < n; i++) s += (double)v[i] * v[i];
    return n ? sqrt(s / (double)n) : 0.0;
}

double qko_max_rel_err(const float *got, const float *ref, size_t n)
{
    const double rms = rms_of(ref, n);
    const double floor_d = fmax(1e-3, 1e-3 * rms);
    double worst = 0;
    for (size_t i = 0; i < n; i++) {
        const double den = fmax(floor_d, fabs((double)ref[i]));
        double rel = fabs((double)got[i] - (double)ref[i]) / den;
        if (isnan(rel)) rel = INFINITY;
        if (rel > worst) worst = rel;
    }
    return worst;
}

double qko_max_err_over_rms(const float *got, const float *ref, size_t n)
{
    const double rms = rms_of(ref, n);
    double worst = 0;
    for (size_t i = 0; i < n; i++) {
        double e = fabs((double)got[i] - (double)ref[i]);
        if (isnan(e)) e = INFINITY;
        if (e > worst) worst = e;
    }
    return rms > 0 ? worst / rms : worst;
}

/* ---- layer glue ---------------------------------------------------------------- */
/* v = a [+ b [+ c]] in float, left to right, as the shaders form it
 * (shaders/add_rmsnorm.comp:28, add_rms3.comp:29); the norm as the CPU checker computes it,
 * in double: sc = 1/sqrt(sum(v^2)/n + eps), xn = (float)(v * sc * w) (src/main.cpp:1685-1690). */
void qko_add_rms(const float *a, const float *b, const float *c, const float *w, float *sum_out,
                 float *xn, uint32_t n, float eps)
{
    double ss = 0;
    for (uint32_t i = 0; i < n; i++) {
        float v = a[i];
        if (b) v = v + b[i];
        if (c) v = v + c[i];
        ss += (double)v * v;
    }
    const double sc = 1.0 / sqrt(ss / n + eps);
    for (uint32_t i = 0; i < n; i++) {
        float v = a[i];
        if (b) v = v + b[i];
        if (c) v = v + c[i];
        if (sum_out) sum_out[i] = v;
        xn[i] = (float)(v * sc * w[i]);
    }
}

/* x[r] = dequantised row ids[idx + per_req*r] of W [n_vocab][kdim]
 * (shaders/embed_q6k.comp:27-49, embed_q8_0.comp:24-34). */
int qko_embed(int type, const void *W, uint32_t n_vocab, uint32_t kdim, const uint32_t *ids,
              uint32_t idx, uint32_t per_req, float *x, uint32_t rows)
{
    const size_t rb = qko_row_bytes(type, kdim);
    if (!rb) return -1;
    for (uint32_t r = 0; r < rows; r++) {
        const uint32_t tok = ids[idx + per_req * r];
        if (tok >= n_vocab) return -2;
        if (qko_dequant_row(type, (const uint8_t *)W + (size_t)tok * rb, x + (size_t)r * kdim, kdim)) return -1;
    }
    return 0;
}
