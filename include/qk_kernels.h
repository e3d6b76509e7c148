/* qk_kernels.h -- operator-level C ABI of libqk.so (MI355X / gfx950).
 *
 * The reference has no exported per-kernel API: each of its kernels is a compute
 * pipeline with a fixed contract -- storage buffers in binding order, a small
 * push-constant block, the dispatch z axis as the slot/token index -- consumed by
 * makePipe()/disp() (reference src/main.cpp:779-816, 4186-4193).  This header states
 * those contracts as plain C entry points over device pointers so the engine, the
 * benchmark and the tests drive the kernels without a model file.  Each function
 * cites the reference pipeline(s) it stands for (paths relative to the reference tree).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless its name ends in _host;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream); all work
 *    is enqueued on it and nothing synchronises unless stated;
 *  - weights are raw GGUF blocks, row-major, rows of K elements, tensor base aligned
 *    to 16 bytes; activations and outputs are fp32;
 *  - return 0 on success, a negative QKK_E* code otherwise; qkk_last_error() returns
 *    the message of the calling thread's last failure;
 *  - there is no CPU fallback: without a HIP device every compute entry point fails
 *    with QKK_EDEVICE.
 */
#ifndef QK_KERNELS_H
#define QK_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QKK_MAX_SLOTS 16u   /* decode slots per step (reference include/qk.h:21) */
#define QKK_MAX_USED 16u    /* picks per token (reference shaders/moe_select.comp:8) */
#define QKK_MAX_EXPERTS 512u

/* ggml tensor type ids (reference src/gguf.h:17-21) */
enum qkk_type {
    QKK_F32 = 0,
    QKK_F16 = 1,
    QKK_Q8_0 = 8,
    QKK_Q6_K = 14,
    QKK_IQ3_XXS = 18,
    QKK_IQ4_XS = 23,
};

enum qkk_status {
    QKK_OK = 0,
    QKK_EINVAL = -1,   /* null pointer, zero size, misaligned tensor */
    QKK_ESHAPE = -2,   /* shape the kernels do not cover (K not a block multiple, ...) */
    QKK_ETYPE = -3,    /* tensor type not supported by this entry point */
    QKK_EDEVICE = -4,  /* no HIP device / launch failure */
    QKK_EWORKSPACE = -5 /* workspace too small */
};

/* Router output of one slot, 160 bytes: the SelT every MoE pipeline binds
 * (reference shaders/moe_select.comp:15). */
typedef struct qkk_sel {
    uint32_t ids[16];
    float w[16];
    float w_shared;
    float pad[7];
} qkk_sel;

/* One MoE layer's device tensors (reference src/main.cpp:1258-1263, MoeT). */
typedef struct qkk_moe_layer {
    uint32_t n_embd, n_ff, n_expert, n_used;
    int32_t gu_type;   /* QKK_IQ3_XXS */
    int32_t down_type; /* QKK_IQ4_XS or QKK_Q6_K */
    const float *gate_inp;       /* [n_expert][n_embd] f32 */
    const float *gate_inp_shexp; /* [n_embd] f32 */
    const void *gate_exps;       /* [n_expert][n_ff] rows of n_embd */
    const void *up_exps;         /* [n_expert][n_ff] rows of n_embd */
    const void *down_exps;       /* [n_expert][n_embd] rows of n_ff */
    const void *gate_shexp;      /* Q8_0 [n_ff] rows of n_embd */
    const void *up_shexp;        /* Q8_0 [n_ff] rows of n_embd */
    const void *down_shexp;      /* Q8_0 [n_embd] rows of n_ff */
} qkk_moe_layer;

const char *qkk_last_error(void);

/* Library / device probe. Returns the number of HIP devices (0 when none), fills
 * arch_host (e.g. "gfx950") when non-NULL. Never fails. */
int qkk_device_info(char *arch_host, size_t arch_len, uint32_t *n_cu_host);

/* Switches between two forms of the same operator (no counterpart in the reference, whose pipelines
 * are chosen when they are built: reference src/main.cpp:3630-3760).  Each is read once from the
 * environment variable QK_<NAME> on first use; qkk_set_option changes it for the calling process
 * (launches already captured in a graph keep the form they were captured with).  Names and values:
 *   "one_row"     0 (env "lane", the default): the one-row GEMV, MoE step and LM head load block
 *                 fields per lane; 1 (env "stream"): they stream rows as 16-byte pieces through LDS
 *   "dense_reg"   1: the F16 / F32 GEMV keeps its share of x in registers
 *   "fused_norm"  1: the engine's one-row step folds each RMS norm into its consumer
 *   "attn_block"  1: prefill attention over blocks of 16 rows on the matrix cores
 *   "dn_fused"    1: the gated-DeltaNet decode step as one launch
 *   "gemm_tiled"  1: products with 64 and more activation rows (qkk_gemm_q8_0, qkk_gemv) decode every
 *                 weight tile once per 128 rows instead of once per 32
 *   "moe_rows"    1: the routed experts' projections for more than ten rows (qkk_moe_decode, qkk_moe_prefill)
 *                 with each wave owning 16 weight rows for all of K, instead of the waves splitting K
 *   "head_rows"   1: qkk_head_argmax for 2..16 rows with each wave owning 16 vocabulary rows for all of K
 *   "select_ranked" (default 1; matters with "one_row" = 1 only) 0: the streamed gate/up launch picks the experts
 *                 in n_used rounds on one wave, as the per-lane form does, instead of by rank counting on four
 *   "gemv_depth", "head_depth", "rowwise_max": launch-shape sweeps, 0 = built-in value
 * The default of every switch is the form that has been run and timed on a device.
 * Returns QKK_EINVAL for an unknown name or a value outside the switch's range. */
int qkk_set_option(const char *name_host, int value);
int qkk_get_option(const char *name_host, int *value_host);

/* Bytes of one row of k elements of `type`; 0 if unsupported (reference src/gguf.h:36-46). */
size_t qkk_row_bytes(int type, uint64_t k);

/* out[i] = fp32 value of element i of a block stream, evaluated in the reference's
 * order with no contraction, so the result is bit-identical to its CPU dequantisation
 * (reference src/quants.h:70-165). Debug / verification kernel. n_elems must be a
 * multiple of the block size. */
int qkk_dequant(int type, const void *W, float *out, uint64_t n_elems, void *stream);

/* Y[b][m] = W[m] . X[b], b < batch <= 16.  Stands for gemv_{f16,q8_0,q6_k,iq4_xs,iq3_xxs}.comp
 * (reference shaders/gemv_q8_0.comp:29-71, gemv_q6_k.comp:35-96, gemv_iq4_xs.comp:34-77,
 * gemv_iq3_xxs.comp:30-78, gemv_f16.comp:21-44) and, for QKK_F32, moe_logits.comp:18-37.
 * X is [batch][K], Y is [batch][M]. */
int qkk_gemv(int type, const void *W, const float *X, float *Y, uint32_t M, uint32_t K,
             uint32_t batch, void *stream);

/* The same product with the RMS norm of the activation row in front and no launch of its own:
 * Y[b][m] = W[m] . (X[b] * w_norm / sqrt(mean(X[b]^2) + eps)).  Stands for rmsnorm.comp followed by the
 * gemv_*.comp dispatches that read the normalised row (reference src/main.cpp:4307-4335: attn_norm, then
 * the mixer's input projections).  Quantised block formats, K = 2048, batch <= 16 (one pass over the
 * weights per row). */
int qkk_gemv_norm(int type, const void *W, const float *X, const float *w_norm, float eps, float *Y,
                  uint32_t M, uint32_t K, uint32_t batch, void *stream);

/* Workspace for qkk_moe_decode with up to n_slots slots. */
size_t qkk_moe_workspace_bytes(const qkk_moe_layer *L_host, uint32_t n_slots);

/* Fused MoE step for n_slots activation rows (reference src/main.cpp:4379-4402 without
 * the residual/RMS half of add_rms3): router logits, top-n_used select and softmax over
 * the picks, sigmoid shared gate, routed gate/up with SiLU, routed down, shared expert,
 * weighted combine.  Stands for moe_logits / moe_select / moe_gateup_iq3 / moe_gateup_q8 /
 * moe_down_{iq4,q6k} / moe_down_q8b and the a+b sum of add_rms3.comp:27-31.
 *   X   [n_slots][n_embd]          in
 *   Y   [n_slots][n_embd]          out: routed + shared contribution (no residual)
 *   sel [n_slots]                  out: picks in pick order, weights, shared gate
 *   workspace                      qkk_moe_workspace_bytes(), 256-byte aligned, must be
 *                                  zero-filled once before its first use (a fill issued on
 *                                  another stream must have completed, or `stream` must wait
 *                                  for it); calls sharing a workspace must not overlap in
 *                                  time.  A workspace that breaks this gives wrong results,
 *                                  never an access outside the tensors: the kernels clamp
 *                                  every index they take from it.
 * With n_slots > QKK_ROWWISE_MAX every picked expert's weights are read once per 16 rows that picked
 * it (matrix-core path); that path needs n_embd = 2048 and returns QKK_ESHAPE otherwise. */
int qkk_moe_decode(const qkk_moe_layer *L_host, const float *X, float *Y, qkk_sel *sel,
                   void *workspace, size_t workspace_bytes, uint32_t n_slots, void *stream);

/* Waits for `stream` and says whether a routing launch since the last such call found a workspace whose
 * header was not zero -- never cleared, or cleared on another stream that had not finished: with more
 * than QKK_ROWWISE_MAX rows the step then counts its workgroups' arrivals from garbage, and its results
 * are invalid (inside the tensors, but wrong).  QKK_OK, or QKK_EINVAL once per occurrence (the flag is
 * per device and cleared by the call that reports it).  The reference's dispatches need no such state
 * (a command buffer's barriers order them); this is the check for this library's one-time zero-fill
 * contract.  Synchronises: for set-up code, tests and debug builds, not for a serving loop. */
int qkk_moe_workspace_status(void *stream);

/* qkk_moe_decode without a workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The workspace is a device array of QKK_MOE_STATIC_BYTES inside the
 * library (one copy per device, held until the process ends); the entry point calls no hipMalloc,
 * hipFree or other allocating routine.  Same kernels, same results bit for bit as qkk_moe_decode.
 *   n_slots <= QKK_MOE_STATIC_MAX_SLOTS; a layer shape whose workspace exceeds the array is refused
 *   with QKK_EWORKSPACE (n_embd 2048, n_ff 512, 256 experts, 8 picks, 16 rows need 1.5 MB).
 * Every call on a device shares that device's array: calls that overlap in time on one device race,
 * whatever their streams.  The array's address is resolved on the first call on a device (or by
 * qkk_device_info); make that call outside a stream capture. */
#define QKK_MOE_STATIC_MAX_SLOTS 16u
#define QKK_MOE_STATIC_BYTES (2u << 20)
int qkk_moe_decode_static(const qkk_moe_layer *L_host, const float *X, float *Y, qkk_sel *sel,
                          uint32_t n_slots, void *stream);

/* The step followed by the layer tail (reference src/main.cpp:4379-4402 with add_rms3.comp:24-41,
 * for several rows add_rms3_grouped.comp:22-50):
 *   S[r]  = resid[r] + (routed + shared contribution of row r)    the next layer's residual input
 *   Xn[r] = S[r] * w_next / sqrt(mean(S[r]^2) + eps)              normalised with the NEXT layer's weight
 * X, sel, workspace, n_slots as for qkk_moe_decode.  resid may be S (in place); Xn must be a buffer
 * of its own.  Above QKK_ROWWISE_MAX rows the tail runs inside the launch that sums the experts'
 * slots, so the step's output is never written on its own; up to that many rows it costs one more
 * small launch (qkk_moe_layer_rows spends none). */
int qkk_moe_decode_tail(const qkk_moe_layer *L_host, const float *X, const float *resid,
                        const float *w_next, float eps, float *S, float *Xn, qkk_sel *sel,
                        void *workspace, size_t workspace_bytes, uint32_t n_slots, void *stream);

/* Rows up to which qkk_moe_decode / qkk_moe_decode_tail run every row through the one-row launches
 * (a few rows hardly ever pick the same expert, so there is little to share, and a row's result is
 * then bit for bit what it is alone); more rows take the expert-major path. */
#define QKK_ROWWISE_MAX 10u

/* One whole MoE block of a layer for n_slots <= QKK_ROWWISE_MAX activation rows, norm in front and
 * residual behind (reference src/main.cpp:4376-4402: the norm half of add_rmsnorm.comp, the MoE
 * stages, the sum of add_rms3.comp), in place on the residual rows S [n_slots][n_embd]:
 *   xn = S * w_norm / sqrt(mean(S^2) + eps);   S <- S + (routed + shared contribution of xn)
 * No launch is spent on the norm or the add: a dot product against xn is 1/rms(S) times the dot
 * product against S * w_norm, so the router and gate/up launches form S * w_norm once per workgroup
 * while summing the squares and scale their sums; the down launch adds the residual to its outputs.
 * Three launches.  sel, workspace as for qkk_moe_decode.  More rows: QKK_ESHAPE, use
 * qkk_moe_decode_tail. */
int qkk_moe_layer_rows(const qkk_moe_layer *L_host, float *S, const float *w_norm, float eps, qkk_sel *sel,
                       void *workspace, size_t workspace_bytes, uint32_t n_slots, void *stream);

/* The same with a mixer's output on top of the residual (reference src/main.cpp:4376-4402 with the
 * add half of add_rmsnorm.comp too):  T <- S + mix;  S <- T + (contribution of norm(T)).
 * The first launch adds while it loads (and stores T [n_slots][n_embd], a buffer of its own, for the
 * other two), so the add + norm launch between mixer and MoE block is not needed.  Results are bit
 * for bit those of qkk_moe_layer_rows on rows added beforehand. */
int qkk_moe_layer_rows_add(const qkk_moe_layer *L_host, float *S, const float *mix, float *T,
                           const float *w_norm, float eps, qkk_sel *sel, void *workspace,
                           size_t workspace_bytes, uint32_t n_slots, void *stream);

/* The same step cut at its launch boundaries, for per-stage timing (the reference times its
 * MoE stages separately under QK_STEP_PROF, src/main.cpp:4173-4185, 4591-4632).  `stages` is
 * a mask of QKK_STAGE_*; a stage reads what the earlier stages of a previous call left in
 * sel / workspace.  With all three stages it is the three-launch form of the step. */
#define QKK_STAGE_ROUTE 1u  /* router logits, shared gate/up, select   */
#define QKK_STAGE_GATEUP 2u /* routed gate/up + SiLU                     */
#define QKK_STAGE_DOWN 4u   /* routed + shared down, weighted combine    */
#define QKK_STAGE_ALL 7u
int qkk_moe_decode_stages(const qkk_moe_layer *L_host, const float *X, float *Y, qkk_sel *sel,
                          void *workspace, size_t workspace_bytes, uint32_t n_slots, uint32_t stages,
                          void *stream);

/* Counting sort of (token, pick) pairs by expert (reference shaders/moe_group_pairs.comp:19-51):
 * offsets[n_expert+1], pairs[n_tokens*n_used] = (token<<4)|pick, ascending inside an expert. */
int qkk_moe_group_pairs(const qkk_sel *sel, uint32_t n_tokens, uint32_t n_expert, uint32_t n_used,
                        uint32_t *offsets, uint32_t *pairs, void *stream);

/* LM head + greedy sample (reference src/main.cpp:4406-4419: gemv_q6_k TPR=128, argmax1.comp,
 * argmax2.comp): tok[b] = argmax_m W[m] . X[b], ties to the lower id.  W is Q6_K [V][K].
 * logits (optional, [batch][V]) receives the fp32 logits when non-NULL.
 * workspace: qkk_head_workspace_bytes(V, batch) bytes, zero-filled once before first use. */
size_t qkk_head_workspace_bytes(uint32_t V, uint32_t batch);
int qkk_head_argmax(const void *W, const float *X, uint32_t *tok, float *logits, uint32_t V,
                    uint32_t K, uint32_t batch, void *workspace, size_t workspace_bytes,
                    void *stream);

/* The same for ONE row with the output norm in front and no launch of its own: tok[0] = argmax_m
 * W[m] . (X * w_norm / sqrt(mean(X^2) + eps)) (reference src/main.cpp:4406-4419: rmsnorm.comp with
 * output_norm, then the head's GEMV and the argmax pair).  K = 2048. */
int qkk_head_argmax_norm(const void *W, const float *X, const float *w_norm, float eps, uint32_t *tok,
                         float *logits, uint32_t V, uint32_t K, void *workspace,
                         size_t workspace_bytes, void *stream);

/* Two-pass argmax over fp32 rows (reference shaders/argmax1.comp:17-40, argmax2.comp:16-30):
 * tok[b] = first index of the maximum of logits[b][0..n). */
int qkk_argmax(const float *logits, uint32_t *tok, uint32_t n, uint32_t batch, void *stream);

/* Batched-prefill dense projection Y[n][m] = X[n] . W[m], W in Q8_0 (reference
 * shaders/gemm_q8_0.comp:32-101, gemm_q8_0_coopmat2.comp:42-148): Q8_0 rows streamed through
 * LDS, MFMA on half operands with fp32 accumulation (activations and weights kept exact to
 * ~2^-22 by hi/lo splits).  X [N][K] fp32, Y [N][M] fp32, K a multiple of 32. */
int qkk_gemm_q8_0(const void *W, const float *X, float *Y, uint32_t M, uint32_t K, uint32_t N,
                  void *stream);

/* Batched-prefill MoE for n_tokens rows (reference src/main.cpp:5050-5198: moe_logits_gemm,
 * moe_select, moe_group_pairs, moe_gateup_iq3_grouped_coopmat, moe_down_*_grouped_coopmat,
 * moe_gateup_q8_coopmat, moe_down_q8_coopmat, the routed fold of add_rms3_grouped.comp:22-27).
 * Same tensors and outputs as qkk_moe_decode, n_tokens <= 4096. */
size_t qkk_moe_prefill_workspace_bytes(const qkk_moe_layer *L_host, uint32_t n_tokens);
int qkk_moe_prefill(const qkk_moe_layer *L_host, const float *X, float *Y, qkk_sel *sel,
                    void *workspace, size_t workspace_bytes, uint32_t n_tokens, void *stream);

/* ---- layer glue: the fp32 steps between the projections of a layer ---------------------------
 * Rows are activation rows (the reference's z = slot), n floats each, contiguous.  Outputs may be
 * the inputs (in place); w must not overlap an output.  eps >= 0 (the reference passes 1e-6,
 * src/main.cpp:4194).
 *   qkk_rmsnorm      out = x * scale * w,  scale = 1/sqrt(mean(x^2) + eps)
 *                    (reference shaders/rmsnorm.comp:19-32)
 *   qkk_add_rmsnorm  y = a + b;  xn = y * scale(y) * w   (residual add + the layer's FFN norm;
 *                    reference shaders/add_rmsnorm.comp:23-40; add_rmsnorm_route.comp is the same
 *                    arithmetic plus a counter reset this library does not need)
 *   qkk_add_rms3     s = (a + b) + c;  xn = s * scale(s) * w   (layer tail: residual + routed +
 *                    shared, normalised with the NEXT layer's weight; reference
 *                    shaders/add_rms3.comp:24-41).  qkk_moe_decode already returns routed + shared
 *                    as one row, so a caller of this library uses qkk_add_rmsnorm for the tail.
 *   qkk_vec_add      out = a + b   (reference shaders/vec_add.comp:13-14) */
int qkk_rmsnorm(const float *x, const float *w, float *out, uint32_t n, uint32_t rows, float eps,
                void *stream);
int qkk_add_rmsnorm(const float *a, const float *b, const float *w, float *y, float *xn, uint32_t n,
                    uint32_t rows, float eps, void *stream);
int qkk_add_rms3(const float *a, const float *b, const float *c, const float *w, float *s, float *xn,
                 uint32_t n, uint32_t rows, float eps, void *stream);
int qkk_vec_add(const float *a, const float *b, float *out, uint64_t n, void *stream);

/* Embedding lookup (reference shaders/embed_q6k.comp:27-49, embed_q8_0.comp:24-34; the reference
 * dispatches Q6_K or Q8_0, src/main.cpp:3678): x[r][0..kdim) = the dequantised row
 * ids[idx + per_req * r] of the token-embedding tensor W [n_vocab][kdim], r < rows; bit-identical
 * to qkk_dequant of that row.  ids is a device array of n_ids token ids; an id >= n_vocab reads
 * the last row. */
int qkk_embed(int type, const void *W, uint32_t n_vocab, uint32_t kdim, const uint32_t *ids,
              uint32_t n_ids, uint32_t idx, uint32_t per_req, float *x, uint32_t rows, void *stream);

/* ---- full-attention mixer, decode step ---------------------------------------------------------
 * (reference shaders/fa_prep_srv.comp:26-76, fa_attn_srv.comp:27-95 and its split / grouped forms
 * fa_attn_srv_split_gqa.comp, fa_attn_srv_reduce.comp; host src/main.cpp:4246-4300; CPU mirror
 * src/main.cpp:2138-2201.)  Head size dh = 256; hQ query heads on hKV KV heads, hQ/hKV <= 8.
 *   qfull    [slots][hQ][2*dh]   per head dh query values, then dh output-gate pre-activations
 *   kin, vin [slots][hKV][dh]
 *   caches   [slots][hKV][tmax][dh] fp32
 *   rope     [tmax][n_rot/2][2] (cos, sin) on the device; qkk_rope_table fills a host array the
 *            way the reference does (src/main.cpp:2011-2020, float powf / cosf / sinf)
 *   slot_pos [slots] device words: position of the slot's new token (clamped to tmax - 1)
 * qkk_attn_prep: per head RMS norm with q_norm_w / k_norm_w, the first n_rot dims rotated by the
 *   position's angles (pairs j, j + n_rot/2); queries to qhat [slots][hQ][dh], keys and values into
 *   the caches at slot_pos.
 * qkk_attn_decode: att[slot][h] = softmax(qhat[h] . K[0..pos] / sqrt(dh)) V[0..pos] * sigmoid(gate),
 *   K/V of KV head h / (hQ/hKV).  Every cache row is read once for the hQ/hKV heads that share it;
 *   positions are cut into 8..64 ranges that run in parallel and are folded in range order.  The
 *   launch shape depends on the slot count and tmax only, so a captured graph stays valid as
 *   positions advance.
 *   workspace: qkk_attn_workspace_bytes(), 256-byte aligned, no initialisation needed. */
int qkk_rope_table(float *rope_host, uint32_t tmax, uint32_t n_rot, float freq_base);
int qkk_attn_prep(const float *qfull, const float *kin, const float *vin, const float *q_norm_w,
                  const float *k_norm_w, const float *rope, const uint32_t *slot_pos, float *qhat,
                  float *k_cache, float *v_cache, uint32_t n_slots, uint32_t hQ, uint32_t hKV, uint32_t dh,
                  uint32_t n_rot, uint32_t tmax, float eps, void *stream);
size_t qkk_attn_workspace_bytes(uint32_t n_slots, uint32_t hQ, uint32_t dh);
int qkk_attn_decode(const float *qhat, const float *k_cache, const float *v_cache, const float *qfull,
                    const uint32_t *slot_pos, float *att, void *workspace, size_t workspace_bytes,
                    uint32_t n_slots, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax, void *stream);

/* ---- gated-DeltaNet mixer, decode step ----------------------------------------------------------
 * (reference shaders/dn_ab.comp:20-50, dn_convn.comp:20-54, dn_step_gate.comp:26-81 = dn_step.comp
 * + dn_gate.comp; host src/main.cpp:4200-4244; CPU mirror src/main.cpp:1704-1768.)  State size
 * dS = 128; hK query/key heads, hV value heads; channels = (2*hK + hV) * dS, q heads first, then k,
 * then v.
 * qkk_dn_ab    gb[slot][h]      = a_vec[h] * softplus(alpha_w[h] . x[slot] + dt_bias[h])   (log decay)
 *              gb[slot][hV + h] = sigmoid(beta_w[h] . x[slot])                             (write strength)
 *              alpha_w, beta_w F32 [hV][n_embd]; n_embd 2048 or 4096.
 * qkk_dn_conv  out[slot][ch] = silu(st0*ker[ch][0] + st1*ker[ch][1] + st2*ker[ch][2] + qkv[slot][ch]*ker[ch][3]),
 *              conv_state [slots][channels][3] shifted (oldest first); the heads below qk_channels
 *              are then scaled by 1 / max(|head|, eps).
 * qkk_dn_step  per value head h, with kh = h / kdiv (kdiv = 0: h % hK, the reference's two pairings,
 *              src/main.cpp:3092-3094), decay = exp(gb[h]), beta = gb[hV + h]:
 *                sk_j = decay * sum_i S[j][i] k_i;  d_j = beta * (v_j - sk_j);
 *                S[j][i] <- S[j][i] * decay + k_i * d_j;  o_j = sum_i S[j][i] q_i / sqrt(dS);
 *                att[slot][h][j] = o_j / sqrt(mean_j o_j^2 + eps) * norm_w[j] * silu(z[slot][h][j])
 *              state [slots][hV][dS][dS] fp32, COLUMN-major per head: element (row j, column i) at
 *              [i][j] (a wave then reads consecutive floats; the reference keeps it row-major).
 *              Bound by the state: dS*dS*4 bytes read and written per head. */
int qkk_dn_ab(const float *x, const float *alpha_w, const float *beta_w, const float *dt_bias,
              const float *a_vec, float *gb, uint32_t n_embd, uint32_t hV, uint32_t n_slots, void *stream);
int qkk_dn_conv(float *conv_state, const float *qkv, const float *ker, float *out, uint32_t channels,
                uint32_t d_state, uint32_t qk_channels, float eps, uint32_t n_slots, void *stream);
/* qkk_dn_ab and qkk_dn_conv in one launch (neither reads what the other writes; the same results
 * bit for bit): for decode steps, where two launches of a few microseconds are mostly launch ramp. */
int qkk_dn_ab_conv(const float *x, const float *alpha_w, const float *beta_w, const float *dt_bias,
                   const float *a_vec, float *gb, uint32_t n_embd, uint32_t hV, float *conv_state,
                   const float *qkv, const float *ker, float *out, uint32_t channels, uint32_t d_state,
                   uint32_t qk_channels, float eps, uint32_t n_slots, void *stream);
/* qkk_dn_ab_conv with x the residual row: the RMS norm in front of the mixer (weights w_norm, norm_eps)
 * is applied to x on the way into the alpha / beta dot products (n_embd 2048), so a one-row decode step
 * needs no norm launch (the projections that feed qkv take the norm the same way: qkk_gemv_norm). */
int qkk_dn_ab_conv_norm(const float *x, const float *w_norm, float norm_eps, const float *alpha_w,
                        const float *beta_w, const float *dt_bias, const float *a_vec, float *gb,
                        uint32_t n_embd, uint32_t hV, float *conv_state, const float *qkv, const float *ker,
                        float *out, uint32_t channels, uint32_t d_state, uint32_t qk_channels, float eps,
                        uint32_t n_slots, void *stream);
int qkk_dn_step(const float *conv, const float *gb, float *state, const float *norm_w, const float *z,
                float *att, uint32_t d_state, uint32_t hK, uint32_t hV, uint32_t kdiv, float eps,
                uint32_t n_slots, void *stream);
/* The decode step of the mixer in ONE launch: qkk_dn_ab_conv (with the norm in front when w_norm is given,
 * NULL otherwise) and qkk_dn_step, same arithmetic in the same order, same results bit for bit; conv and gb
 * never touch memory.  A workgroup takes the two value heads of one key head (they share the q / k conv
 * window, which is shifted once), so hV = 2 hK is required (the reference's 32 on 16; kdiv 0 or 2),
 * n_embd 2048.  conv_state [slots][(2 hK + hV) dS][3], qkv [slots][(2 hK + hV) dS]. */
int qkk_dn_step_fused(const float *x, const float *w_norm, float norm_eps, const float *alpha_w,
                      const float *beta_w, const float *dt_bias, const float *a_vec, uint32_t n_embd,
                      float *conv_state, const float *qkv, const float *ker, float *state,
                      const float *norm_w, const float *z, float *att, uint32_t d_state, uint32_t hK,
                      uint32_t hV, uint32_t kdiv, float eps, uint32_t n_slots, void *stream);

/* ---- the mixers over consecutive positions of ONE slot (prompt prefill) ---------------------------
 * (reference shaders/fa_prep_batch.comp, fa_attn_batch.comp, dn_conv_batch.comp, dn_step_batch.comp
 * + dn_gate_batch.comp; host src/main.cpp:3953-4090.)  Rows are positions base, base+1, ... of one
 * slot; conv_state, state and the caches are that slot's alone.  Results per position are those of
 * the decode-step entry points called position by position.
 * qkk_attn_prep_seq  row t is written into the caches at positions[t] (distinct, ascending).
 * qkk_attn_seq       row t attends to the cache rows 0..positions[t]: causal over the rows of this
 *                    call and everything the cache held before.  Three or more rows: a scan blocked
 *                    over 16 rows and 4 query heads per workgroup, scores and values on the matrix
 *                    cores (reference shaders/fa_attn_batch_coopmat.comp:58-183); two rows share one
 *                    scan of the cache.  workspace: qkk_attn_workspace_bytes(n_pos, hQ, dh).
 * qkk_dn_conv_seq    the conv is a 4-tap filter over the inputs, so all positions run in parallel
 *                    (bit-identical to the steps); the window is moved on by a second small launch.
 * qkk_dn_step_seq    the state is read once, kept in registers over all positions (8 rows of a head
 *                    per workgroup, 16 lanes per row) and written once; q, k, v and the gates are
 *                    staged through LDS 16 positions at a time; the head norm and output gate run
 *                    as a second launch over (head, position).  conv 16-byte aligned, n_pos <= 65535. */
int qkk_attn_prep_seq(const float *qfull, const float *kin, const float *vin, const float *q_norm_w,
                      const float *k_norm_w, const float *rope, const uint32_t *positions, float *qhat,
                      float *k_cache, float *v_cache, uint32_t n_pos, uint32_t hQ, uint32_t hKV,
                      uint32_t dh, uint32_t n_rot, uint32_t tmax, float eps, void *stream);
int qkk_attn_seq(const float *qhat, const float *k_cache, const float *v_cache, const float *qfull,
                 const uint32_t *positions, float *att, void *workspace, size_t workspace_bytes,
                 uint32_t n_pos, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax, void *stream);
int qkk_dn_conv_seq(float *conv_state, const float *qkv, const float *ker, float *out, uint32_t channels,
                    uint32_t d_state, uint32_t qk_channels, float eps, uint32_t n_pos, void *stream);
int qkk_dn_step_seq(const float *conv, const float *gb, float *state, const float *norm_w, const float *z,
                    float *att, uint32_t d_state, uint32_t hK, uint32_t hV, uint32_t kdiv, float eps,
                    uint32_t n_pos, void *stream);

#ifdef __cplusplus
}
#endif
#endif
