// qk_engine.cpp -- engine-level C ABI (include/qk.h).
//
// The reference engine runs a whole hybrid model; this library implements the quantized
// decode hot path only (GEMVs, fused MoE step, LM head, prefill GEMMs -- see qk_kernels.h).
// qk_open() therefore validates its arguments with the reference's limits and messages
// (reference src/main.cpp:3575, 5396-5402) and then reports that a whole-model engine
// cannot be built from the kernels present.  Every other entry point keeps the
// reference's argument checks and return codes (reference src/main.cpp:5405-5532) so a
// host that resolves the full symbol set loads this library unchanged.
#include <stdio.h>

#include <new>
#include <vector>

#include "../../include/qk.h"

struct qk_engine {
    uint32_t n_slots = 0, n_ctx = 0, chunk = 0;
    uint32_t vocab = 0, eos = 0, bos = 0;
    uint32_t layer_first = 0, layer_end = 0, n_layer = 0, n_embd = 2048;
    uint32_t n_state = 0;
    bool split = false;
    struct Slot { bool active = false; };
    std::vector<Slot> slots;
};

static void set_err(char* err, size_t n, const char* msg)
{
    if (err && n) snprintf(err, n, "%s", msg);
}

extern "C" {

qk_engine* qk_open(const char* gguf_path, const qk_config* cfg, char* err, size_t err_len)
{
    if (!gguf_path || !cfg) { set_err(err, err_len, "qk_open: null arg"); return nullptr; }
    if (cfg->n_slots < 1 || cfg->n_slots > 16 || cfg->n_ctx < 64 || cfg->n_ctx > 65536 || cfg->chunk < 1 ||
        cfg->chunk > 32) {
        set_err(err, err_len, "qk_open: bad config");
        return nullptr;
    }
    FILE* f = fopen(gguf_path, "rb");
    if (!f) {
        set_err(err, err_len, "qk_open: cannot open GGUF");
        return nullptr;
    }
    fclose(f);
    set_err(err, err_len,
            "qk_open: this libqk.so implements the quantized decode hot path only (see qk_kernels.h); "
            "the attention / gated-DeltaNet mixers a whole-model engine needs are not part of it");
    return nullptr;
}

void qk_close(qk_engine* e) { delete e; }

uint32_t qk_n_vocab(const qk_engine* e) { return e ? e->vocab : 0; }
uint32_t qk_n_ctx(const qk_engine* e) { return e ? e->n_ctx : 0; }
uint32_t qk_n_slots(const qk_engine* e) { return e ? e->n_slots : 0; }
uint32_t qk_chunk(const qk_engine* e) { return e ? e->chunk : 0; }
uint32_t qk_eos_token(const qk_engine* e) { return e ? e->eos : 0; }
uint32_t qk_bos_token(const qk_engine* e) { return e ? e->bos : 0; }
uint32_t qk_layer_first(const qk_engine* e) { return e ? e->layer_first : 0; }
uint32_t qk_layer_end(const qk_engine* e) { return e ? e->layer_end : 0; }
uint32_t qk_n_layer(const qk_engine* e) { return e ? e->n_layer : 0; }
uint32_t qk_n_embd(const qk_engine* e) { return e ? e->n_embd : 0; }

int qk_slot_start(qk_engine* e, uint32_t slot, const uint32_t* prompt, uint32_t n_prompt, uint32_t max_gen,
                  uint32_t /*snap_prefix*/)
{
    if (!e || slot >= e->n_slots) return -1;
    if (e->split) return -5;
    if (e->slots[slot].active) return -2;
    if (!prompt || n_prompt < 1 || (uint64_t)n_prompt + max_gen > e->n_ctx) return -3;
    for (uint32_t i = 0; i < n_prompt; i++)
        if (prompt[i] >= e->vocab) return -4;
    return -1; // unreachable while qk_open cannot build an engine
}

void qk_slot_cancel(qk_engine* e, uint32_t slot)
{
    if (e && slot < e->n_slots) e->slots[slot].active = false;
}

int qk_step_chunk(qk_engine* e, uint32_t* out_tokens, uint32_t* out_counts, uint32_t* out_finished)
{
    if (!e || !out_tokens || !out_counts || !out_finished) return -1;
    if (e->split) return -5;
    for (uint32_t s = 0; s < e->n_slots; s++) out_counts[s] = 0;
    *out_finished = 0;
    return 0;
}

int qk_stage_run(qk_engine* e, uint32_t slot, const uint32_t* toks, const float* hidden_in, uint32_t n,
                 uint32_t /*base*/, float* hidden_out, uint32_t* ids_out)
{
    if (!e) return -1;
    if (slot >= e->n_slots || n == 0) return -1;
    const bool first = e->layer_first == 0, last = e->layer_end == e->n_layer;
    if (first ? (!toks || hidden_in) : !hidden_in) return -2;
    if (last ? !ids_out : !hidden_out) return -3;
    return -1;
}

int qk_stage_topk(qk_engine* e, uint32_t k, uint32_t* ids, float* vals)
{
    if (!e || k < 1 || k > 256 || !ids || !vals) return -1;
    return -2; // no last-stage run has happened
}

uint32_t qk_state_n(const qk_engine* e) { return e ? e->n_state : 0; }
int qk_state_save(qk_engine* e, uint32_t slot, uint32_t idx, uint32_t)
{
    if (!e || slot >= e->n_slots || idx >= e->n_state) return -1;
    return -1;
}
int qk_state_load(qk_engine* e, uint32_t slot, uint32_t idx, uint32_t)
{
    if (!e || slot >= e->n_slots || idx >= e->n_state) return -1;
    return -1;
}

} // extern "C"
