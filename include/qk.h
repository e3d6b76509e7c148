/* qk.h -- engine-level C ABI of libqk.so.
 *
 * Declarations are those of the reference's include/qk.h (reference include/qk.h:18-125),
 * kept name for name and argument for argument so that a host that dlopen()s the
 * reference library (reference server/src/ffi.rs:120-167) resolves the same symbols here.
 *
 * Threading: every function is called from one engine thread; nothing is thread-safe;
 * qk_step_chunk blocks that thread for one chunk of device steps.
 *
 * State of this build: the engine entry points validate their arguments and report errors
 * exactly as the reference does, but qk_open() cannot run a whole model yet -- the
 * attention and gated-DeltaNet mixers between the MoE blocks are outside the path this
 * library implements -- so it fails with a message saying so.  The kernels of the path
 * (GEMVs, fused MoE step, LM head + argmax, prefill GEMMs) are reached through
 * qk_kernels.h.
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
