/* qk_oracle.h -- CPU oracle for the quantized-weight decode hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a scalar restatement of the reference's
 * CPU checker (its dequantisation header and the inline CPU references of its
 * self-checking CLI modes).  It is linked by the tests, by the smoke check and
 * by the cpu_baseline leg of the benchmark -- never by the product library.
 *
 * Every function names the reference lines it follows (paths relative to
 * /root/reference).  How each function is pinned is listed in qk_oracle.c's
 * header comment.
 */
#ifndef QK_ORACLE_H
#define QK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type ids (src/gguf.h:17-21). */
enum {
    QKO_F32 = 0,
    QKO_F16 = 1,
    QKO_Q8_0 = 8,
    QKO_Q6_K = 14,
    QKO_IQ3_XXS = 18,
    QKO_IQ4_XS = 23,
};

/* Router output of one slot: 160 bytes, the layout every MoE shader binds
 * (shaders/moe_select.comp:15). */
typedef struct qko_sel {
    uint32_t ids[16];
    float w[16];
    float w_shared;
    float pad[7];
} qko_sel;

/* Double-precision router result of the CPU reference (src/main.cpp:1310-1314). */
typedef struct qko_sel_f64 {
    uint32_t ids[16];
    double w[16];
    double w_shared;
    double gap; /* logit[pick k-1] - logit[best non-picked]: margin of the top-k set */
} qko_sel_f64;

/* One MoE layer's tensors (src/main.cpp:1258-1263). Rows are raw GGUF blocks. */
typedef struct qko_moe_layer {
    uint32_t n_embd, n_ff, n_expert, n_used;
    int32_t gu_type;   /* QKO_IQ3_XXS or QKO_IQ4_XS */
    int32_t down_type; /* QKO_IQ4_XS or QKO_Q6_K */
    const float *gate_inp;       /* [n_expert][n_embd] f32 */
    const float *gate_inp_shexp; /* [n_embd] f32 */
    const void *gate_exps;       /* [n_expert][n_ff] rows of n_embd */
    const void *up_exps;         /* [n_expert][n_ff] rows of n_embd */
    const void *down_exps;       /* [n_expert][n_embd] rows of n_ff */
    const void *gate_shexp;      /* Q8_0 [n_ff] rows of n_embd */
    const void *up_shexp;        /* Q8_0 [n_ff] rows of n_embd */
    const void *down_shexp;      /* Q8_0 [n_embd] rows of n_ff */
} qko_moe_layer;

/* src/quants.h:12-48 */
float qko_f16_to_f32(uint16_t h);
uint16_t qko_f32_to_f16(float f);
/* i | parity(i) << 7  (shaders/iq_tables.glsl:2,43; table at src/quant_tables.h:40-49) */
uint8_t qko_ksign(uint32_t i);

/* src/gguf.h:36-46; 0 for an unsupported type or a K the block size does not divide. */
size_t qko_row_bytes(int type, uint64_t k);

/* src/quants.h:70-165 (+ F16/F32 rows, src/main.cpp:645-653). Returns 0, or -1 on bad type/k. */
int qko_dequant_row(int type, const void *row, float *y, int64_t k);

/* y[b][m] = sum_k dequant(W[m])[k] * x[b][k], accumulated in double, rounded to
 * float once (src/main.cpp:626-633, 673-679). scratch: k floats. */
int qko_gemv(int type, const void *W, const float *x, float *y, uint32_t M, uint32_t K,
             uint32_t batch);

/* Greedy sample: first index of the maximum, strict '>' (src/main.cpp:5387-5388). */
uint32_t qko_argmax(const float *v, uint32_t n);

/* Top-k over double logits as the CPU reference does (src/main.cpp:1326-1341);
 * equal logits resolve to the lower id, the rule the GPU selector fixes
 * (shaders/moe_select.comp:53-59). */
void qko_select_f64(const double *logits, uint32_t n_expert, uint32_t n_used, qko_sel_f64 *out);

/* Selector exactly as the device kernel specifies it, in float: non-finite
 * logits become -3.4e38, lower id wins ties, ids clamped, weights
 * exp(l-l0)/sum in pick order (shaders/moe_select.comp:28-34, 53-76). */
void qko_select_f32(const float *logits, uint32_t n_expert, uint32_t n_used, qko_sel *out);

/* Whole fused MoE step for one activation row (src/main.cpp:1316-1387).
 * y: n_embd floats.  sel / h / logits may be NULL.  h: (n_used+1)*n_ff floats,
 * routed experts in pick order then the shared expert
 * (shaders/moe_gateup_iq3.comp:41, moe_gateup_q8.comp:61). logits: n_expert doubles. */
int qko_moe_ref(const qko_moe_layer *L, const float *x, float *y, qko_sel_f64 *sel, float *h,
                double *logits);

/* Counting sort of (token, pick) pairs by expert (shaders/moe_group_pairs.comp:19-51).
 * offsets: n_expert+1; pairs: n_tokens*n_used entries (token<<4)|pick, ascending
 * inside each expert (the shader leaves that order open). */
int qko_group_pairs(const qko_sel *sel, uint32_t n_tokens, uint32_t n_expert, uint32_t n_used,
                    uint32_t *offsets, uint32_t *pairs);

/* Y[n][m] = sum_k X[n][k] * dequant_q8_0(W[m])[k] in double (src/main.cpp:5561-5570). */
int qko_gemm_q8_0(const void *W, const float *X, float *Y, uint32_t M, uint32_t K, uint32_t N);

/* The same row loops on n_threads host threads (qk_oracle_mt.c): bit for bit the results of the
 * single-threaded functions above; for the benchmark's all-cores CPU baseline. */
int qko_gemv_mt(int type, const void *W, const float *x, float *y, uint32_t M, uint32_t K, uint32_t batch,
                uint32_t n_threads);
int qko_gemm_q8_0_mt(const void *W, const float *X, float *Y, uint32_t M, uint32_t K, uint32_t N, uint32_t n_threads);
int qko_moe_ref_mt(const qko_moe_layer *L, const float *x, float *y, uint32_t n_threads);
int qko_moe_ref_tokens_mt(const qko_moe_layer *L, const float *X, float *Y, uint32_t n_tokens, uint32_t n_threads);

/* Scale-aware acceptance metric of the CLI self checks (src/main.cpp:548-565):
 * max over i of |got-ref| / max(|ref|, max(1e-3, 1e-3*rms(ref))). */
double qko_max_rel_err(const float *got, const float *ref, size_t n);

/* max|got-ref| / rms(ref): the batched-GEMM acceptance metric (src/main.cpp:5653-5662). */
double qko_max_err_over_rms(const float *got, const float *ref, size_t n);

/* v = a [+ b [+ c]] in float (b, c may be NULL; shaders/add_rmsnorm.comp:28, add_rms3.comp:29),
 * sum_out (optional) = v, xn = (float)(v * sc * w) with sc = 1/sqrt(sum(v^2)/n + eps) in double
 * (src/main.cpp:1685-1690). */
void qko_add_rms(const float *a, const float *b, const float *c, const float *w, float *sum_out,
                 float *xn, uint32_t n, float eps);

/* Embedding lookup (shaders/embed_q6k.comp:27-49). Returns 0, -1 bad type/kdim, -2 id out of range. */
int qko_embed(int type, const void *W, uint32_t n_vocab, uint32_t kdim, const uint32_t *ids,
              uint32_t idx, uint32_t per_req, float *x, uint32_t rows);

#ifdef __cplusplus
}
#endif
#endif
