/* qk.h -- engine-level C ABI of libqk.so.
 *
 * Declarations are those of the reference's include/qk.h (reference include/qk.h:18-125),
 * kept name for name and argument for argument so that a host that dlopen()s the
 * reference library (reference server/src/ffi.rs:120-167) resolves the same symbols here.
 *
 * Threading: every function is called from one engine thread; nothing is thread-safe;
 * qk_step_chunk blocks that thread for one chunk of device steps.
 *
 * What qk_open() runs:
 *   - a whole-model GGUF of the reference's family: token embedding, per layer attn_norm + a mixer
 *     (gated DeltaNet where "ssm_a" is present, else full attention) + post_attention_norm + the
 *     eight MoE tensors, output_norm, Q6_K head; head shapes as in the reference engine (DeltaNet
 *     32 value / 16 key heads of 128, attention 16 x 256 query heads on 2 KV heads, n_embd 2048);
 *     dense projections Q8_0 or IQ4_XS; ssm_alpha / ssm_beta as separate F32 tensors, or fused as
 *     ssm_ba (F32, Q8_0 or IQ4_XS; reference src/main.cpp:3931-3948): split on the device at open);
 *   - a GGUF whose layers are MoE blocks only (no mixer tensors at all).
 * Every entry point behaves as the reference's: argument checks and return codes, the serial-step
 * state machine of qk_step_chunk (one captured hipGraph per dispatch depth), greedy sampling,
 * EOS / max_gen / n_ctx endings, qk_stage_run / qk_stage_topk on the unsplit engine, state
 * snapshots (three entries, or QK_PCACHE).  qk_slot_start prefills the positions the reference batch-prefills,
 * and qk_stage_run feeds its positions, in passes of up to QK_PREFILL_ROWS rows on the slot
 * alone.  Not part of this library: the prefix cache, speculative decoding, QK_LAYERS pipeline
 * stages (refused: one GPU runs every layer).  A device failure inside a call returns -6.
 * Environment, as in the reference: QK_MAXB (batch-prefill chunk, 16..1024, default 128),
 * QK_NO_BATCH (serial prefill of the whole prompt), QK_PCACHE (state snapshot entries, 1..256, default 3);
 * and QK_PREFILL_ROWS (rows of one prefill
 * pass, 16..1024, default 1024: how the prefilled positions are cut, not which are prefilled),
 * QK_NO_GRAPH (launch the step's kernels one by one instead of replaying the graph), QK_WEIGHT_SLAB=1 (the file's
 * tensors carved from one device allocation instead of one each);
 * QK_STEP_PROF, as in the reference (src/main.cpp:4591-4632): the first decode step of slot 0 alone is launched
 * kernel by kernel with an event behind every stage and the stages' times go to stderr once
 * ("[prof] decode step: ... us on-GPU across N stages", one line per stage name; QK_STEP_PROF_DETAIL adds every
 * interval in launch order); QK_COUNTERS (src/main.cpp:5250-5281): the same for the first prefill pass of more
 * than one row ("[qk counters] HIP batched prefill N=... span=... ms", one line per stage; QK_COUNTER_RAW adds
 * every interval).
 */
#ifndef QK_H
#define QK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qk_engine qk_engine;

/* reference include/qk.h:20-24 */
typedef struct qk_config {
    uint32_t n_slots; /* concurrent sequences, 1..16 */
    uint32_t n_ctx;   /* tokens per slot (prompt + generated), 64..65536 */
    uint32_t chunk;   /* device steps per host sync, 1..32 */
} qk_config;

/* reference include/qk.h:28-30.  NULL on failure; err (if err_len > 0) always ends in NUL. */
qk_engine *qk_open(const char *gguf_path, const qk_config *cfg, char *err, size_t err_len);
void qk_close(qk_engine *e);

/* reference include/qk.h:32-37 */
uint32_t qk_n_vocab(const qk_engine *e);
uint32_t qk_n_ctx(const qk_engine *e);
uint32_t qk_n_slots(const qk_engine *e);
uint32_t qk_chunk(const qk_engine *e);
uint32_t qk_eos_token(const qk_engine *e);
uint32_t qk_bos_token(const qk_engine *e);

/* reference include/qk.h:39-51; error codes reference src/main.cpp:5449-5453:
 * -1 bad engine/slot, -2 slot busy, -3 bounds or null prompt, -4 token >= vocab,
 * -5 engine is a pipeline stage. The prompt is copied. */
int qk_slot_start(qk_engine *e, uint32_t slot, const uint32_t *prompt, uint32_t n_prompt,
                  uint32_t max_gen, uint32_t snap_prefix);

/* reference include/qk.h:53-55.  Safe on a free slot. */
void qk_slot_cancel(qk_engine *e, uint32_t slot);

/* reference include/qk.h:57-72.  out_tokens: n_slots*chunk u32, slot s writes at
 * [s*chunk, s*chunk+out_counts[s]); out_finished: bit s set when slot s ended (EOS is not
 * emitted).  Returns the number of slots active at entry, -1 on null arguments, -5 on a
 * pipeline-stage engine (reference src/main.cpp:5528-5531). */
int qk_step_chunk(qk_engine *e, uint32_t *out_tokens, uint32_t *out_counts, uint32_t *out_finished);

/* reference include/qk.h:87-90 */
uint32_t qk_layer_first(const qk_engine *e);
uint32_t qk_layer_end(const qk_engine *e);
uint32_t qk_n_layer(const qk_engine *e);
uint32_t qk_n_embd(const qk_engine *e);

/* reference include/qk.h:92-106; -1/-2/-3 on bad arguments (reference src/main.cpp:5294-5296). */
int qk_stage_run(qk_engine *e, uint32_t slot, const uint32_t *toks, const float *hidden_in, uint32_t n,
                 uint32_t base, float *hidden_out, uint32_t *ids_out);

/* reference include/qk.h:108-114; -1 bad arguments, -2 no run yet (reference src/main.cpp:5314-5315). */
int qk_stage_topk(qk_engine *e, uint32_t k, uint32_t *ids, float *vals);

/* reference include/qk.h:116-131; -1 on bad arguments. */
uint32_t qk_state_n(const qk_engine *e);
int qk_state_save(qk_engine *e, uint32_t slot, uint32_t idx, uint32_t n_tok);
int qk_state_load(qk_engine *e, uint32_t slot, uint32_t idx, uint32_t n_tok);

#ifdef __cplusplus
}
#endif
#endif /* QK_H */
