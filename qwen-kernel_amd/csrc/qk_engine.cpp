// qk_engine.cpp -- engine-level C ABI (include/qk.h): the slot state machine of the reference
// engine (reference src/main.cpp:4462-4666 stepChunk, 5447-5532 slot start / cancel / step)
// over the kernels of this library, one hipGraph per dispatch depth in place of the
// reference's pre-recorded command buffers (reference src/main.cpp:4186-4422).
//
// What the engine can run.  The reference model alternates a mixer (full attention or gated
// DeltaNet) with a MoE block in every layer.  qk_open() takes
//   - a whole-model file: per layer  xn = rmsnorm(x, attn_norm); y = x + mixer(xn);
//     x = y + MoE(rmsnorm(y, post_attention_norm))  -- the reference's decode step
//     (src/main.cpp:4194-4405) from this library's operators; per-slot state stripes (conv window
//     and delta-rule state, or K / V cache) live in the engine;
//   - a file whose layers are MoE blocks only: the same step with every mixer output zero; such a
//     model keeps no per-position state.
//   token' = argmax(output.weight . rmsnorm(x, output_norm)), Q6_K head, ties to the lower id.
// Everything the host sees -- argument checks, return codes, which step emits which token,
// EOS / max_gen / n_ctx endings, the finished mask -- follows the reference line by line.  The
// positions the reference batch-prefills at qk_slot_start are fed here one token at a time on the
// starting slot alone (no batched-prefill kernels for the mixers); prefix cache and speculative
// decoding are not part of this library.
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <initializer_list>
#include <new>
#include <string>
#include <utility>
#include <vector>

#include "../../include/qk.h"
#include "../../include/qk_gguf.h"
#include "qk_host.h"

namespace {

constexpr uint32_t N_EMBD = 2048;           // reference src/main.cpp:3086 (compile-time there too)
constexpr uint32_t MAX_ROWS = QKK_MAX_SLOTS; // rows one device step carries
constexpr uint32_t N_STATE_DEFAULT = 3;     // snapshot entries (reference default, stub/qk_stub.c:98; QK_PCACHE sets 1..256, src/main.cpp:4121-4125)
constexpr int ERR_DEVICE = -6;              // a launch, copy or synchronisation failed

// The mixers' shapes are fixed, as in the reference engine (src/main.cpp:3085-3090).
constexpr uint32_t DN_CH = 8192, DN_IN = 4096, DN_HV = 32, DN_DS = 128, DN_HK = 16; // gated DeltaNet
constexpr uint32_t FA_DH = 256, FA_HQ = 16, FA_HKV = 2, FA_ROT = 64;                // full attention
constexpr float FA_FREQ_BASE = 1e7f;                                                // src/main.cpp:1872

struct Dense { // a Q8_0 / IQ4_XS projection [M][K]
    const void* w = nullptr;
    int type = 0;
    uint32_t M = 0, K = 0;
};

struct EngineLayer {
    enum Kind { MOE_ONLY, RECURRENT, ATTENTION };
    Kind kind = MOE_ONLY;
    qkk_moe_layer moe;
    const float* post_norm = nullptr; // blk.l.post_attention_norm.weight
    const float* attn_norm = nullptr; // blk.l.attn_norm.weight (layers with a mixer)
    Dense p1, p2, p3, out;            // recurrent: attn_qkv, attn_gate, -, ssm_out; attention: attn_q, attn_k, attn_v, attn_output
    Dense cat;                        // p1, p2 (, p3) as one matrix when they share a type and lie back to back (else w = null)
    const float *alpha_w = nullptr, *beta_w = nullptr, *dt_bias = nullptr, *a_vec = nullptr, *ker = nullptr,
                *ssm_norm = nullptr;                  // recurrent
    const float *q_norm = nullptr, *k_norm = nullptr; // attention
    float *st1 = nullptr, *st2 = nullptr; // per-slot state: recurrent conv window + delta-rule state; attention K + V cache
    size_t ps1 = 0, ps2 = 0;              // floats per slot of st1 / st2
};

} // namespace

struct qk_engine {
    uint32_t n_slots = 0, n_ctx = 0, chunk = 0;
    uint32_t vocab = 0, eos = 248046, bos = 248044; // reference src/main.cpp:3084
    uint32_t n_layer = 40, layer_first = 0, layer_end = 0;
    uint32_t max_b = 128; // batch-prefill chunk width (reference src/main.cpp:3833)
    int embd_type = 0;
    uint32_t embd_rows = 0;
    float eps = 1e-6f; // reference src/main.cpp:1434

    // device side
    hipStream_t st = nullptr;
    std::vector<void*> dev_allocs;
    // QK_WEIGHT_SLAB=1: the tensors of the file are carved from ONE allocation instead of one each (whether many
    // separate mappings cost the one-row step address translations is a question for a device; default off)
    uint8_t* slab = nullptr;
    size_t slab_bytes = 0, slab_used = 0;
    const void* d_embd = nullptr;
    const void* d_head = nullptr;
    const float* d_onorm = nullptr;
    std::vector<EngineLayer> layers;
    uint32_t* d_ids = nullptr;  // [MAX_ROWS] tokens fed this step
    uint32_t* d_tok = nullptr;  // [MAX_ROWS] tokens sampled this step
    float* d_x = nullptr;       // [MAX_ROWS][N_EMBD] residual stream
    float* d_xn[2] = {nullptr, nullptr}; // normalised rows, alternating between layers
    float* d_last = nullptr;    // [N_EMBD] final normalised row of the last stage run
    float* d_logits = nullptr;  // [vocab]
    qkk_sel* d_sel = nullptr;
    void* d_ws = nullptr;
    size_t ws_bytes = 0;
    void* d_hws = nullptr;
    size_t hws_bytes = 0;
    uint32_t* h_ids = nullptr; // pinned, [MAX_ROWS]
    uint32_t* h_tok = nullptr; // pinned, [MAX_ROWS]
    std::vector<hipGraphExec_t> graphs; // [depth - 1], empty when graphs are switched off
    uint32_t last_run_rows = 0;
    // whole-model files (layers with mixers)
    bool full_model = false;
    uint32_t dn_kdiv = 0;        // 0: value head h reads key head h % hK; else h / dn_kdiv (src/main.cpp:3092-3094)
    uint32_t* d_pos = nullptr;   // [MAX_ROWS] position of the token fed this step
    uint32_t* h_pos = nullptr;   // pinned
    uint32_t pf_rows = 1024;     // positions of one slot a prefill pass carries (whole-model files; QK_PREFILL_ROWS)
    uint32_t cap = MAX_ROWS;     // rows the step's buffers hold (pf_rows for whole-model files)
    bool cat_everywhere = false; // every layer's input projections lie back to back (one product per layer)
    bool fused_norm = false;     // the "fused_norm" switch at qk_open: every consumer of a normalised row of the one-row step normalises on the way in
    bool dn_one_launch = false;  // the "dn_fused" switch at qk_open: the gated-DeltaNet decode step as one launch (to be measured against two)
    uint32_t *d_pf = nullptr, *h_pf = nullptr; // [3][pf_rows] ids, positions, sampled ids of a prefill pass (device / pinned)
    float* d_rope = nullptr;     // [n_ctx][FA_ROT/2][2]
    float *d_big = nullptr, *d_mid = nullptr, *d_kin = nullptr, *d_vin = nullptr, *d_gb = nullptr, *d_conv = nullptr,
          *d_qhat = nullptr, *d_att = nullptr, *d_mix = nullptr; // per-step rows of the mixers
    void* d_aws = nullptr;       // attention workspace
    size_t aws_bytes = 0;
    uint32_t n_state = N_STATE_DEFAULT;     // snapshot entries (QK_PCACHE)
    std::vector<std::vector<float*>> snaps; // [n_state][2 * layer]: one slot's state stripes
    // QK_STEP_PROF (reference src/main.cpp:3300-3305, 4591-4632): the first pure decode step at depth 1 is launched
    // kernel by kernel with an event behind every stage, and the stages' times are printed once to stderr
    bool prof_on = false, prof_armed = false, prof_printed = false;
    // QK_COUNTERS (reference src/main.cpp:3307-3313, 5250-5281): the same for the first prefill pass of more than one row
    bool counters_on = false, counters_printed = false;
    std::vector<std::pair<const char*, hipEvent_t>> prof_ev;
    void stamp(const char* label);
    void prof_report();
    void counters_report(uint32_t rows, uint32_t base);

    // host side (reference src/main.cpp:3153-3175, Slot)
    struct Slot {
        bool active = false;
        std::vector<uint32_t> prompt;
        uint32_t cursor = 0, pos = 0, last = 0, gen = 0, max_gen = 0;
    };
    std::vector<Slot> slots;

    ~qk_engine();
    bool open(const char* path, const qk_config& cfg, char* err, size_t err_len);
    bool upload(const qkg_tensor& t, const void** out, char* err, size_t err_len);
    void* dev_alloc(size_t bytes, bool zero);
    void dev_free(const void* p); // a staging buffer of qk_open that nothing refers to any more
    int launch_rows(uint32_t rows, float** final_rows);
    int launch_full(uint32_t rows, uint32_t s0, float** final_rows, bool want_head, bool seq);
    int prefill(uint32_t slot, const uint32_t* toks, uint32_t n, uint32_t base, uint32_t* ids_out);
    int reset_slot(uint32_t slot);
    bool load_mixers(qkg_file* g, char* err, size_t err_len);
    int copy_state(uint32_t slot, uint32_t idx, bool save, uint32_t n_tok);
    int run_rows(uint32_t rows, bool graph_ok);
    int copy_and_launch(uint32_t rows);
    int step_chunk(uint32_t* out_tok, uint32_t* out_cnt, uint32_t* out_fin);
    int stage_run(uint32_t slot, const uint32_t* toks, const float* hidden_in, uint32_t n, uint32_t base,
                  float* hidden_out, uint32_t* ids_out);
    int stage_topk(uint32_t k, uint32_t* ids, float* vals);
    bool split() const { return layer_first != 0 || layer_end != n_layer; }
};

static bool set_err(char* err, size_t n, const char* msg)
{
    if (err && n) snprintf(err, n, "%s", msg);
    return false;
}

qk_engine::~qk_engine()
{
    if (st) (void)hipStreamSynchronize(st);
    for (auto& p : prof_ev) (void)hipEventDestroy(p.second);
    for (hipGraphExec_t g : graphs)
        if (g) (void)hipGraphExecDestroy(g);
    for (void* p : dev_allocs) (void)hipFree(p);
    if (h_ids) (void)hipHostFree(h_ids);
    if (h_tok) (void)hipHostFree(h_tok);
    if (h_pos) (void)hipHostFree(h_pos);
    if (h_pf) (void)hipHostFree(h_pf);
    if (st) (void)hipStreamDestroy(st);
}

// Device memory the engine owns until it closes, 256 spare bytes behind it; nullptr on failure.
void qk_engine::dev_free(const void* p)
{
    if (slab && (const uint8_t*)p >= slab && (const uint8_t*)p < slab + slab_bytes) return; // carved from the slab: stays until close
    for (size_t i = 0; i < dev_allocs.size(); i++)
        if (dev_allocs[i] == p) {
            (void)hipFree(dev_allocs[i]);
            dev_allocs.erase(dev_allocs.begin() + (long)i);
            return;
        }
}

void* qk_engine::dev_alloc(size_t bytes, bool zero)
{
    void* p = nullptr;
    const size_t take = (bytes + 256 + 255) & ~(size_t)255; // the slab hands out 256-byte aligned pieces, the spare bytes included
    if (slab && slab_used + take <= slab_bytes) {
        p = slab + slab_used;
        slab_used += take;
        if (zero && hipMemset(p, 0, bytes + 256) != hipSuccess) return nullptr;
        return p;
    }
    if (hipMalloc(&p, bytes + 256) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    dev_allocs.push_back(p);
    if (zero && hipMemset(p, 0, bytes + 256) != hipSuccess) return nullptr;
    return p;
}

// Copies one tensor of the file into device memory of its own (256 spare bytes behind it).
bool qk_engine::upload(const qkg_tensor& t, const void** out, char* err, size_t err_len)
{
    uint8_t* p = (uint8_t*)dev_alloc(t.nbytes, false);
    if (!p) return set_err(err, err_len, "qk_open: device memory exhausted");
    if (hipMemcpy(p, t.data, t.nbytes, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemset(p + t.nbytes, 0, 256) != hipSuccess)
        return set_err(err, err_len, "qk_open: upload failed");
    *out = p;
    return true;
}

// The launches of one device step over `rows` rows: d_ids -> d_tok.  *final_rows receives the
// buffer that holds the rows normalised with output_norm (the LM head's input).
// An event behind what has been launched so far, named for the stage it closes (only while the profiled step runs).
void qk_engine::stamp(const char* label)
{
    if (!prof_armed) return;
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return;
    if (hipEventRecord(e, st) != hipSuccess) { (void)hipEventDestroy(e); return; }
    prof_ev.emplace_back(label, e);
}

// The profiled step has been waited for: per stage name the launches, their time and their share, longest first
// (the reference's lines, src/main.cpp:4609-4615; QK_STEP_PROF_DETAIL adds every interval in launch order).
void qk_engine::prof_report()
{
    struct Row { const char* name; uint32_t n; double us; };
    std::vector<Row> rows;
    std::vector<double> each;
    double total = 0;
    for (size_t i = 1; i < prof_ev.size(); i++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, prof_ev[i - 1].second, prof_ev[i].second) != hipSuccess) ms = 0.f;
        const double us = (double)ms * 1e3;
        each.push_back(us);
        total += us;
        auto it = std::find_if(rows.begin(), rows.end(), [&](const Row& r) { return !strcmp(r.name, prof_ev[i].first); });
        if (it == rows.end()) rows.push_back(Row{prof_ev[i].first, 1, us});
        else { it->n++; it->us += us; }
    }
    std::sort(rows.begin(), rows.end(), [](const Row& a, const Row& b) { return a.us > b.us; });
    fprintf(stderr, "[prof] decode step: %.0f us on-GPU across %zu stages\n", total, each.size());
    for (const Row& r : rows)
        fprintf(stderr, "[prof]   %-10s n=%-3u tot=%8.1f us  avg=%6.2f us  %4.1f%%\n", r.name, r.n, r.us, r.us / r.n,
                total > 0 ? 100.0 * r.us / total : 0.0);
    if (getenv("QK_STEP_PROF_DETAIL")) {
        uint32_t layer = 0;
        for (size_t i = 1; i < prof_ev.size(); i++) {
            fprintf(stderr, "[prof-detail] seq=%-3zu layer=%-2u %-10s %8.2f us\n", i, layer, prof_ev[i].first, each[i - 1]);
            if (!strcmp(prof_ev[i].first, "moe") || !strcmp(prof_ev[i].first, "moe+tail")) layer++;
        }
    }
    for (auto& p : prof_ev) (void)hipEventDestroy(p.second);
    prof_ev.clear();
}

// The profiled prefill pass has been waited for: per stage name its time, share and launches, in launch order
// (the reference's lines, src/main.cpp:5276-5281; QK_COUNTER_RAW adds every interval).
void qk_engine::counters_report(uint32_t rows, uint32_t base)
{
    struct Agg { const char* name; double ms; uint32_t count; };
    std::vector<Agg> agg;
    double total = 0;
    for (size_t i = 1; i < prof_ev.size(); i++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, prof_ev[i - 1].second, prof_ev[i].second) != hipSuccess) ms = 0.f;
        total += ms;
        auto it = std::find_if(agg.begin(), agg.end(), [&](const Agg& a) { return !strcmp(a.name, prof_ev[i].first); });
        if (it == agg.end()) agg.push_back(Agg{prof_ev[i].first, ms, 1});
        else { it->ms += ms; it->count++; }
        if (getenv("QK_COUNTER_RAW")) fprintf(stderr, "[qk counter raw] %03zu %-22s %9.3f ms\n", i, prof_ev[i].first, ms);
    }
    fprintf(stderr, "[qk counters] HIP batched prefill N=%u base=%u span=%.3f ms markers=%zu\n", rows, base, total, prof_ev.size());
    for (const Agg& a : agg)
        fprintf(stderr, "[qk counters] %-22s %9.3f ms %6.2f%%  (%u passes)\n", a.name, a.ms, total > 0 ? 100.0 * a.ms / total : 0.0,
                a.count);
    for (auto& p : prof_ev) (void)hipEventDestroy(p.second);
    prof_ev.clear();
}

int qk_engine::launch_rows(uint32_t rows, float** final_rows)
{
    if (rows < 1 || rows > MAX_ROWS) return QKK_ESHAPE;
    stamp("t0");
    if (int rc = qkk_embed(embd_type, d_embd, embd_rows, N_EMBD, d_ids, MAX_ROWS, 0, 1, d_x, rows, st)) return rc;
    stamp("emb");
    if (rows <= QKK_ROWWISE_MAX) {
        // few rows: each layer's norm runs inside its MoE launches and the residual is added by the
        // last of them -- three launches per layer, then the output norm and the head.  Every row
        // goes through the one-row kernels, so a slot's tokens do not depend on its company.
        for (const EngineLayer& L : layers) {
            if (int rc = qkk_moe_layer_rows(&L.moe, d_x, L.post_norm, eps, d_sel, d_ws, ws_bytes, rows, st)) return rc;
            stamp("moe");
        }
        if (int rc = qkk_rmsnorm(d_x, d_onorm, d_xn[0], N_EMBD, rows, eps, st)) return rc;
        stamp("rms");
        if (final_rows) *final_rows = d_xn[0];
        const int rc = qkk_head_argmax(d_head, d_xn[0], d_tok, nullptr, vocab, N_EMBD, rows, d_hws, hws_bytes, st);
        stamp("head");
        return rc;
    }
    if (int rc = qkk_rmsnorm(d_x, layers[0].post_norm, d_xn[0], N_EMBD, rows, eps, st)) return rc;
    int cur = 0;
    for (size_t l = 0; l < layers.size(); l++) {
        const float* w_next = l + 1 < layers.size() ? layers[l + 1].post_norm : d_onorm;
        if (int rc = qkk_moe_decode_tail(&layers[l].moe, d_xn[cur], d_x, w_next, eps, d_x, d_xn[cur ^ 1], d_sel, d_ws,
                                         ws_bytes, rows, st))
            return rc;
        cur ^= 1;
    }
    if (final_rows) *final_rows = d_xn[cur];
    return qkk_head_argmax(d_head, d_xn[cur], d_tok, nullptr, vocab, N_EMBD, rows, d_hws, hws_bytes, st);
}

static int dense(const Dense& d, const float* x, float* y, uint32_t rows, hipStream_t st)
{
    return qkk_gemv(d.type, d.w, x, y, d.M, d.K, rows, st);
}

// The launches of one pass of a whole model (reference src/main.cpp:4194-4419).
//   seq = false: one decode step over the slots [s0, s0 + rows): d_ids / d_pos -> d_tok.  Every
//                per-slot buffer is indexed from s0, so slots can be stepped apart from the others.
//   seq = true:  `rows` consecutive positions of slot s0 (ids, positions, sampled ids in d_pf): the
//                projections, norms and MoE blocks take all rows at once -- every weight is read once
//                for the pass -- and the mixers run their sequence forms (one launch per kernel:
//                the conv window and the recurrent state stay in registers over the positions,
//                attention is causal over the rows).
int qk_engine::launch_full(uint32_t rows, uint32_t s0, float** final_rows, bool want_head, bool seq)
{
    // the state stripes hold n_slots slots: no pass reaches behind them
    if (rows < 1 || s0 >= n_slots || (seq ? rows > pf_rows : s0 + rows > n_slots)) return QKK_ESHAPE;
    float* x = d_x;
    const uint32_t* ids = seq ? d_pf : d_ids;
    const uint32_t* pos = seq ? d_pf + pf_rows : d_pos + s0;
    uint32_t* tok = seq ? d_pf + 2 * pf_rows : d_tok + s0;
    stamp("t0");
    if (int rc = qkk_embed(embd_type, d_embd, embd_rows, N_EMBD, ids, seq ? pf_rows : MAX_ROWS, seq ? 0 : s0, 1, x, rows, st))
        return rc;
    stamp("emb");
    // One row of a decode step (no caller wants the normalised rows): no norm launches at all.  The
    // consumers of a normalised row -- the input projections, the decay / write-strength products, the
    // head -- take the residual row and the norm's weights and normalise on the way in; the MoE
    // launches have done so all along.
    const bool fuse = rows == 1 && !seq && !final_rows && cat_everywhere && fused_norm;
    if (!fuse) {
        if (int rc = qkk_rmsnorm(x, layers[0].attn_norm, d_xn[0], N_EMBD, rows, eps, st)) return rc;
        stamp("rms0");
    }
    int cur = 0;
    for (size_t l = 0; l < layers.size(); l++) {
        const EngineLayer& L = layers[l];
        float* xn = d_xn[cur];
        float *s1 = L.st1 + s0 * L.ps1, *s2 = L.st2 + s0 * L.ps2;
        // one row: the input projections as one product into d_big, their outputs back to back
        const bool one = rows == 1 && L.cat.w;
        if (fuse) {
            if (int rc = qkk_gemv_norm(L.cat.type, L.cat.w, x, L.attn_norm, eps, d_big, L.cat.M, L.cat.K, 1, st)) return rc;
        } else if (one)
            if (int rc = dense(L.cat, xn, d_big, 1, st)) return rc;
        const bool rec = L.kind == EngineLayer::RECURRENT;
        if (rec) {
            float* d_mid = one ? d_big + DN_CH : this->d_mid;
            if (!one) {
                if (int rc = dense(L.p1, xn, d_big, rows, st)) return rc;
                if (int rc = dense(L.p2, xn, d_mid, rows, st)) return rc;
            }
            stamp("dn.proj");
            if (seq) {
                if (int rc = qkk_dn_ab(xn, L.alpha_w, L.beta_w, L.dt_bias, L.a_vec, d_gb, N_EMBD, DN_HV, rows, st)) return rc;
                if (int rc = qkk_dn_conv_seq(s1, d_big, L.ker, d_conv, DN_CH, DN_DS, 2 * DN_HK * DN_DS, eps, rows, st)) return rc;
                stamp("dn.ab+conv");
                if (int rc = qkk_dn_step_seq(d_conv, d_gb, s2, L.ssm_norm, d_mid, d_att, DN_DS, DN_HK, DN_HV, dn_kdiv, eps, rows,
                                             st))
                    return rc;
            } else if (dn_one_launch) {
                // QK_DN_FUSED=1: ab, conv and step in one launch (a workgroup per key head; the same results bit for bit)
                if (int rc = qkk_dn_step_fused(fuse ? x : xn, fuse ? L.attn_norm : nullptr, eps, L.alpha_w, L.beta_w, L.dt_bias,
                                               L.a_vec, N_EMBD, s1, d_big, L.ker, s2, L.ssm_norm, d_mid, d_att, DN_DS, DN_HK,
                                               DN_HV, dn_kdiv, eps, rows, st))
                    return rc;
            } else {
                // decay / write strength and the conv in one launch
                if (int rc = fuse ? qkk_dn_ab_conv_norm(x, L.attn_norm, eps, L.alpha_w, L.beta_w, L.dt_bias, L.a_vec, d_gb, N_EMBD,
                                                        DN_HV, s1, d_big, L.ker, d_conv, DN_CH, DN_DS, 2 * DN_HK * DN_DS, eps, rows,
                                                        st)
                                  : qkk_dn_ab_conv(xn, L.alpha_w, L.beta_w, L.dt_bias, L.a_vec, d_gb, N_EMBD, DN_HV, s1, d_big,
                                                   L.ker, d_conv, DN_CH, DN_DS, 2 * DN_HK * DN_DS, eps, rows, st))
                    return rc;
                stamp("dn.ab+conv");
                if (int rc = qkk_dn_step(d_conv, d_gb, s2, L.ssm_norm, d_mid, d_att, DN_DS, DN_HK, DN_HV, dn_kdiv, eps, rows, st))
                    return rc;
            }
            stamp("dn.step");
        } else {
            float* d_kin = one ? d_big + FA_HQ * 2 * FA_DH : this->d_kin;
            float* d_vin = one ? d_kin + FA_HKV * FA_DH : this->d_vin;
            if (!one) {
                if (int rc = dense(L.p1, xn, d_big, rows, st)) return rc;
                if (int rc = dense(L.p2, xn, d_kin, rows, st)) return rc;
                if (int rc = dense(L.p3, xn, d_vin, rows, st)) return rc;
            }
            stamp("at.proj");
            if (seq) {
                if (int rc = qkk_attn_prep_seq(d_big, d_kin, d_vin, L.q_norm, L.k_norm, d_rope, pos, d_qhat, s1, s2, rows, FA_HQ,
                                               FA_HKV, FA_DH, FA_ROT, n_ctx, eps, st))
                    return rc;
                stamp("at.prep");
                if (int rc = qkk_attn_seq(d_qhat, s1, s2, d_big, pos, d_att, d_aws, aws_bytes, rows, FA_HQ, FA_HKV, FA_DH, n_ctx,
                                          st))
                    return rc;
            } else {
                if (int rc = qkk_attn_prep(d_big, d_kin, d_vin, L.q_norm, L.k_norm, d_rope, pos, d_qhat, s1, s2, rows, FA_HQ,
                                           FA_HKV, FA_DH, FA_ROT, n_ctx, eps, st))
                    return rc;
                stamp("at.prep");
                if (int rc = qkk_attn_decode(d_qhat, s1, s2, d_big, pos, d_att, d_aws, aws_bytes, rows, FA_HQ, FA_HKV, FA_DH,
                                             n_ctx, st))
                    return rc;
            }
            stamp("at.attn");
        }
        if (int rc = dense(L.out, d_att, d_mix, rows, st)) return rc;
        stamp(rec ? "dn.out" : "at.out");
        const float* w_next = l + 1 < layers.size() ? layers[l + 1].attn_norm : d_onorm;
        if (rows <= QKK_ROWWISE_MAX) {
            // x <- (x + mixer) + MoE(norm(x + mixer)) in three launches (xn, read by now, takes the sum), then
            // the next layer's norm
            if (int rc = qkk_moe_layer_rows_add(&L.moe, x, d_mix, xn, L.post_norm, eps, d_sel, d_ws, ws_bytes, rows, st))
                return rc;
            stamp("moe");
            if (!fuse) {
                if (int rc = qkk_rmsnorm(x, w_next, d_xn[cur ^ 1], N_EMBD, rows, eps, st)) return rc;
                stamp("rms");
            }
        } else {
            // y = x + mixer, normalised for the MoE block; then x = y + MoE, normalised for the next layer
            if (int rc = qkk_add_rmsnorm(x, d_mix, L.post_norm, x, xn, N_EMBD, rows, eps, st)) return rc;
            stamp("addN");
            if (int rc = qkk_moe_decode_tail(&L.moe, xn, x, w_next, eps, x, d_xn[cur ^ 1], d_sel, d_ws, ws_bytes, rows, st))
                return rc;
            stamp("moe+tail");
        }
        cur ^= 1;
    }
    if (final_rows) *final_rows = d_xn[cur];
    if (!want_head) return QKK_OK;
    if (fuse) {
        const int rc = qkk_head_argmax_norm(d_head, x, d_onorm, eps, tok, nullptr, vocab, N_EMBD, d_hws, hws_bytes, st);
        stamp("head");
        return rc;
    }
    for (uint32_t r0 = 0; r0 < rows; r0 += MAX_ROWS) // the head takes sixteen rows at a time
        if (int rc = qkk_head_argmax(d_head, d_xn[cur] + (size_t)r0 * N_EMBD, tok + r0, nullptr, vocab, N_EMBD,
                                     std::min(MAX_ROWS, rows - r0), d_hws, hws_bytes, st))
            return rc;
    stamp("head");
    return QKK_OK;
}

// Positions base .. base+n-1 of one slot, alone (the other slots' states are not touched), in
// passes of pf_rows.  ids_out (optional): the greedy id after every position; the last position's
// normalised row is kept for qk_stage_topk.
int qk_engine::prefill(uint32_t slot, const uint32_t* toks, uint32_t n, uint32_t base, uint32_t* ids_out)
{
    for (uint32_t off = 0; off < n; off += pf_rows) {
        const uint32_t rows = std::min(pf_rows, n - off);
        for (uint32_t t = 0; t < rows; t++) {
            h_pf[t] = toks[off + t];
            h_pf[pf_rows + t] = base + off + t;
        }
        if (hipMemcpyAsync(d_pf, h_pf, 2 * pf_rows * sizeof(uint32_t), hipMemcpyHostToDevice, st) != hipSuccess)
            return ERR_DEVICE;
        float* fin = nullptr;
        const bool trace = counters_on && !counters_printed && rows > 1;
        prof_armed = trace;
        const int rc_pass = launch_full(rows, slot, &fin, ids_out != nullptr, true);
        prof_armed = false;
        if (rc_pass != QKK_OK) return ERR_DEVICE;
        if (ids_out && (hipMemcpyAsync(h_pf + 2 * pf_rows, d_pf + 2 * pf_rows, rows * sizeof(uint32_t), hipMemcpyDeviceToHost,
                                       st) != hipSuccess ||
                        hipMemcpyAsync(d_last, fin + (size_t)(rows - 1) * N_EMBD, N_EMBD * sizeof(float),
                                       hipMemcpyDeviceToDevice, st) != hipSuccess))
            return ERR_DEVICE;
        if (hipStreamSynchronize(st) != hipSuccess) return ERR_DEVICE;
        if (trace) {
            counters_report(rows, base + off);
            counters_printed = true;
        }
        if (ids_out) memcpy(ids_out + off, h_pf + 2 * pf_rows, rows * sizeof(uint32_t));
    }
    return 0;
}

// Clears a slot's recurrent state (reference resetSlot, src/main.cpp:3416-3433); the KV rows of an
// attention layer are overwritten as the positions are fed.
int qk_engine::reset_slot(uint32_t slot)
{
    for (const EngineLayer& L : layers)
        if (L.kind == EngineLayer::RECURRENT &&
            (hipMemsetAsync(L.st1 + slot * L.ps1, 0, L.ps1 * sizeof(float), st) != hipSuccess ||
             hipMemsetAsync(L.st2 + slot * L.ps2, 0, L.ps2 * sizeof(float), st) != hipSuccess))
            return ERR_DEVICE;
    return hipStreamSynchronize(st) == hipSuccess ? 0 : ERR_DEVICE;
}

// One device step: h_ids[0..rows) in, h_tok[0..rows) out, host blocked until it is done.  A
// captured step holds the two copies as well, so a replay is one launch and one wait.
int qk_engine::run_rows(uint32_t rows, bool graph_ok)
{
    if (graph_ok && rows <= graphs.size() && graphs[rows - 1]) {
        if (hipGraphLaunch(graphs[rows - 1], st) != hipSuccess) return ERR_DEVICE;
    } else if (copy_and_launch(rows) != 0) {
        return ERR_DEVICE;
    }
    if (hipStreamSynchronize(st) != hipSuccess) return ERR_DEVICE;
    return 0;
}

int qk_engine::copy_and_launch(uint32_t rows)
{
    if (hipMemcpyAsync(d_ids, h_ids, rows * sizeof(uint32_t), hipMemcpyHostToDevice, st) != hipSuccess)
        return ERR_DEVICE;
    if (full_model) {
        if (hipMemcpyAsync(d_pos, h_pos, rows * sizeof(uint32_t), hipMemcpyHostToDevice, st) != hipSuccess)
            return ERR_DEVICE;
        if (launch_full(rows, 0, nullptr, true, false) != QKK_OK) return ERR_DEVICE;
    } else if (launch_rows(rows, nullptr) != QKK_OK) {
        return ERR_DEVICE;
    }
    if (hipMemcpyAsync(h_tok, d_tok, rows * sizeof(uint32_t), hipMemcpyDeviceToHost, st) != hipSuccess)
        return ERR_DEVICE;
    return 0;
}

// The mixers of a whole-model file (reference src/main.cpp:3916-4010): tensors, per-slot state
// stripes, the step's scratch rows, the RoPE table.  Shapes are the reference's fixed ones.
bool qk_engine::load_mixers(qkg_file* g, char* err, size_t err_len)
{
    auto bad = [&](const char* m) { return set_err(err, err_len, m); };
    auto find = [&](uint32_t l, const char* suffix, qkg_tensor* t) {
        char name[96];
        snprintf(name, sizeof name, "blk.%u.%s", l, suffix);
        return qkg_find(g, name, t) == 0;
    };
    auto f32 = [&](uint32_t l, const char* suffix, uint64_t n_elems, const float** out) {
        qkg_tensor t;
        const void* p = nullptr;
        if (!find(l, suffix, &t) || t.type != QKK_F32 || t.nbytes != n_elems * 4) return false;
        if (!upload(t, &p, err, err_len)) return false;
        *out = (const float*)p;
        return true;
    };
    auto proj = [&](uint32_t l, const char* suffix, uint32_t K, uint32_t M, Dense* d) {
        qkg_tensor t;
        if (!find(l, suffix, &t) || (t.type != QKK_Q8_0 && t.type != QKK_IQ4_XS) || t.ne[0] != K || t.ne[1] != M || !t.nbytes)
            return false;
        d->type = (int)t.type; d->M = M; d->K = K;
        return upload(t, &d->w, err, err_len);
    };
    // The projections that read the same normalised row, uploaded back to back: one row's step
    // runs them as ONE matrix-vector product (their outputs then lie back to back too).
    auto proj_in = [&](uint32_t l, EngineLayer& L, std::initializer_list<std::pair<const char*, uint32_t>> parts) {
        Dense* ds[3] = {&L.p1, &L.p2, &L.p3};
        qkg_tensor ts[3];
        size_t total = 0, n = 0;
        bool same = true;
        for (const auto& pr : parts) {
            qkg_tensor& t = ts[n];
            if (!find(l, pr.first, &t) || (t.type != QKK_Q8_0 && t.type != QKK_IQ4_XS) || t.ne[0] != N_EMBD ||
                t.ne[1] != pr.second || !t.nbytes)
                return false;
            ds[n]->type = (int)t.type; ds[n]->M = pr.second; ds[n]->K = N_EMBD;
            same = same && t.type == ts[0].type && t.nbytes % 16 == 0;
            total += t.nbytes;
            n++;
        }
        if (!same) {
            for (size_t i = 0; i < n; i++)
                if (!upload(ts[i], &ds[i]->w, err, err_len)) return false;
            return true;
        }
        uint8_t* base = (uint8_t*)dev_alloc(total, false);
        if (!base) return set_err(err, err_len, "qk_open: device memory exhausted");
        size_t at = 0;
        for (size_t i = 0; i < n; i++) {
            if (hipMemcpy(base + at, ts[i].data, ts[i].nbytes, hipMemcpyHostToDevice) != hipSuccess)
                return set_err(err, err_len, "qk_open: upload failed");
            ds[i]->w = base + at;
            at += ts[i].nbytes;
            L.cat.M += ds[i]->M;
        }
        if (hipMemset(base + total, 0, 256) != hipSuccess) return set_err(err, err_len, "qk_open: upload failed");
        L.cat.w = base; L.cat.type = ds[0]->type; L.cat.K = N_EMBD;
        return true;
    };
    // qwen3next files hold alpha and beta as ONE tensor ssm_ba [n_embd, 2 * hV] (F32, Q8_0 or IQ4_XS),
    // interleaved per key-head group g: rows 4g, 4g+1 are beta of the value heads 2g, 2g+1, rows 4g+2,
    // 4g+3 their alpha (reference src/main.cpp:3931-3948, which dequantises on the host).  Here the
    // tensor is uploaded as it is, dequantised on the device by the bit-exact kernel and its rows copied
    // apart into the split layout the decay / write-strength kernel reads.
    auto fused_ba = [&](uint32_t l, const float** alpha, const float** beta) {
        qkg_tensor t;
        if (!find(l, "ssm_ba.weight", &t) || t.ne[0] != N_EMBD || t.ne[1] != 2 * DN_HV || !t.nbytes)
            return set_err(err, err_len, "qk_open: missing ssm_alpha/ssm_beta/ssm_ba");
        if (t.type != QKK_F32 && t.type != QKK_Q8_0 && t.type != QKK_IQ4_XS)
            return set_err(err, err_len, "qk_open: ssm_ba type unsupported");
        const uint64_t n_el = 2ull * DN_HV * N_EMBD;
        const void* raw = nullptr;
        if (!upload(t, &raw, err, err_len)) return false;
        const float* rows = (const float*)raw;
        if (t.type != QKK_F32) {
            float* deq = (float*)dev_alloc(n_el * sizeof(float), false);
            if (!deq) return set_err(err, err_len, "qk_open: device memory exhausted");
            if (qkk_dequant((int)t.type, raw, deq, n_el, st) != QKK_OK)
                return set_err(err, err_len, "qk_open: ssm_ba dequantisation failed");
            rows = deq;
        }
        float* al = (float*)dev_alloc((size_t)DN_HV * N_EMBD * sizeof(float), false);
        float* be = (float*)dev_alloc((size_t)DN_HV * N_EMBD * sizeof(float), false);
        if (!al || !be) return set_err(err, err_len, "qk_open: device memory exhausted");
        for (uint32_t r = 0; r < 2 * DN_HV; r++) {
            const uint32_t grp = r >> 2, sub = r & 3;
            float* dst = (sub < 2 ? be : al) + ((size_t)grp * 2 + (sub & 1)) * N_EMBD;
            if (hipMemcpyAsync(dst, rows + (size_t)r * N_EMBD, N_EMBD * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
                return set_err(err, err_len, "qk_open: upload failed");
        }
        if (hipStreamSynchronize(st) != hipSuccess) return set_err(err, err_len, "qk_open: upload failed");
        // the copies are complete: the fused tensor and its dequantised form are not needed again
        if (rows != (const float*)raw) dev_free(rows);
        dev_free(raw);
        *alpha = al; *beta = be;
        return true;
    };
    for (uint32_t l = 0; l < n_layer; l++) {
        EngineLayer& L = layers[l];
        if (!f32(l, "attn_norm.weight", N_EMBD, &L.attn_norm)) return bad("qk_open: missing/unexpected attn_norm tensor");
        if (L.kind == EngineLayer::RECURRENT) {
            if (!proj_in(l, L, {{"attn_qkv.weight", DN_CH}, {"attn_gate.weight", DN_IN}}) ||
                !proj(l, "ssm_out.weight", DN_IN, N_EMBD, &L.out))
                return bad("qk_open: gated-DeltaNet projections missing or of an unsupported type / shape");
            qkg_tensor t_al;
            if (find(l, "ssm_alpha.weight", &t_al)) {
                if (!f32(l, "ssm_alpha.weight", (uint64_t)DN_HV * N_EMBD, &L.alpha_w) ||
                    !f32(l, "ssm_beta.weight", (uint64_t)DN_HV * N_EMBD, &L.beta_w))
                    return bad("qk_open: ssm_alpha/ssm_beta missing or of an unexpected shape");
            } else if (!fused_ba(l, &L.alpha_w, &L.beta_w)) {
                return false;
            }
            if (!f32(l, "ssm_dt.bias", DN_HV, &L.dt_bias) || !f32(l, "ssm_a", DN_HV, &L.a_vec) ||
                !(f32(l, "ssm_conv1d.weight", (uint64_t)DN_CH * 4, &L.ker) || f32(l, "ssm_conv1d", (uint64_t)DN_CH * 4, &L.ker)) ||
                !f32(l, "ssm_norm.weight", DN_DS, &L.ssm_norm))
                return bad("qk_open: gated-DeltaNet tensors missing or of an unexpected shape");
            L.ps1 = (size_t)DN_CH * 3;
            L.ps2 = (size_t)DN_HV * DN_DS * DN_DS;
        } else {
            if (!proj_in(l, L, {{"attn_q.weight", FA_HQ * 2 * FA_DH}, {"attn_k.weight", FA_HKV * FA_DH}, {"attn_v.weight", FA_HKV * FA_DH}}) ||
                !proj(l, "attn_output.weight", FA_HQ * FA_DH, N_EMBD, &L.out))
                return bad("qk_open: attention projections missing or of an unsupported type / shape");
            if (!f32(l, "attn_q_norm.weight", FA_DH, &L.q_norm) || !f32(l, "attn_k_norm.weight", FA_DH, &L.k_norm))
                return bad("qk_open: attention norm tensors missing or of an unexpected shape");
            L.ps1 = L.ps2 = (size_t)FA_HKV * n_ctx * FA_DH;
        }
        L.st1 = (float*)dev_alloc(n_slots * L.ps1 * sizeof(float), true);   // one stripe per configured slot
        L.st2 = (float*)dev_alloc(n_slots * L.ps2 * sizeof(float), true);
        if (!L.st1 || !L.st2) return bad("qk_open: device memory exhausted (per-slot state)");
    }
    auto rows_of = [&](size_t n) { return (float*)dev_alloc(cap * n * sizeof(float), true); };
    d_big = rows_of(DN_CH); d_mid = rows_of(DN_IN); d_kin = rows_of(FA_HKV * FA_DH); d_vin = rows_of(FA_HKV * FA_DH);
    d_gb = rows_of(2 * DN_HV); d_conv = rows_of(DN_CH); d_qhat = rows_of(FA_HQ * FA_DH); d_att = rows_of(DN_IN);
    d_mix = rows_of(N_EMBD);
    d_pos = (uint32_t*)dev_alloc(MAX_ROWS * 4, true);
    d_pf = (uint32_t*)dev_alloc(3 * pf_rows * 4, true);
    if (!d_pf || hipHostMalloc((void**)&h_pf, 3 * pf_rows * 4, hipHostMallocDefault) != hipSuccess)
        return bad("qk_open: cannot allocate the prefill buffers");
    memset(h_pf, 0, 3 * pf_rows * 4);
    aws_bytes = qkk_attn_workspace_bytes(cap, FA_HQ, FA_DH);
    d_aws = dev_alloc(aws_bytes, true);
    d_rope = (float*)dev_alloc((size_t)n_ctx * FA_ROT * sizeof(float), false);
    if (!d_big || !d_mid || !d_kin || !d_vin || !d_gb || !d_conv || !d_qhat || !d_att || !d_mix || !d_pos || !d_aws || !d_rope)
        return bad("qk_open: device memory exhausted");
    std::vector<float> rope((size_t)n_ctx * FA_ROT);
    if (qkk_rope_table(rope.data(), n_ctx, FA_ROT, FA_FREQ_BASE) != QKK_OK ||
        hipMemcpy(d_rope, rope.data(), rope.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
        return bad("qk_open: upload failed");
    // snapshot entries: one slot's state stripes each (reference src/main.cpp:3435-3487, copyStripes)
    snaps.assign(n_state, std::vector<float*>(2 * n_layer, nullptr));
    for (auto& sn : snaps)
        for (uint32_t l = 0; l < n_layer; l++) {
            sn[2 * l] = (float*)dev_alloc(layers[l].ps1 * sizeof(float), true);
            sn[2 * l + 1] = (float*)dev_alloc(layers[l].ps2 * sizeof(float), true);
            if (!sn[2 * l] || !sn[2 * l + 1]) return bad("qk_open: device memory exhausted (snapshots)");
        }
    return true;
}

// Saves a slot's state stripes into snapshot idx, or loads them back.  Of an attention layer's caches
// only the first n_tok positions travel (all of them when n_tok is 0 or beyond n_ctx).
int qk_engine::copy_state(uint32_t slot, uint32_t idx, bool save, uint32_t n_tok)
{
    const uint32_t keep = n_tok == 0 || n_tok > n_ctx ? n_ctx : n_tok;
    for (uint32_t l = 0; l < n_layer; l++) {
        const EngineLayer& L = layers[l];
        float* live[2] = {L.st1 + slot * L.ps1, L.st2 + slot * L.ps2};
        for (int k = 0; k < 2; k++) {
            float* snap = snaps[idx][2 * l + k];
            if (L.kind == EngineLayer::ATTENTION) { // [hKV][n_ctx][dh]: the first `keep` rows of every KV head
                for (uint32_t h = 0; h < FA_HKV; h++) {
                    const size_t off = (size_t)h * n_ctx * FA_DH, n = (size_t)keep * FA_DH * sizeof(float);
                    if (hipMemcpyAsync(save ? snap + off : live[k] + off, save ? live[k] + off : snap + off, n,
                                       hipMemcpyDeviceToDevice, st) != hipSuccess)
                        return ERR_DEVICE;
                }
            } else if (hipMemcpyAsync(save ? snap : live[k], save ? live[k] : snap, (k ? L.ps2 : L.ps1) * sizeof(float),
                                      hipMemcpyDeviceToDevice, st) != hipSuccess) {
                return ERR_DEVICE;
            }
        }
    }
    return hipStreamSynchronize(st) == hipSuccess ? 0 : ERR_DEVICE;
}

bool qk_engine::open(const char* path, const qk_config& cfg, char* err, size_t err_len)
{
    auto bad = [&](const char* m) { return set_err(err, err_len, m); };
    n_slots = cfg.n_slots; n_ctx = cfg.n_ctx; chunk = cfg.chunk;
    // reference src/main.cpp:3575
    if (n_slots < 1 || n_slots > 16 || n_ctx < 64 || n_ctx > 65536 || chunk < 1 || chunk > 32)
        return bad("qk_open: bad config");
    qkg_file* g = qkg_open(path);
    if (!g) return bad("qk_open: cannot open GGUF");
    struct Closer { qkg_file* g; ~Closer() { qkg_close(g); } } closer{g};

    // model shape and token ids (reference src/main.cpp:3580-3590)
    const char* arch_c = "";
    (void)qkg_kv_str(g, "general.architecture", &arch_c);
    const std::string arch = arch_c ? arch_c : "";
    uint64_t v = 0;
    if (qkg_kv_int(g, (arch + ".block_count").c_str(), &v) == 0) n_layer = (uint32_t)v;
    if (n_layer < 1 || n_layer > 256) return bad("qk_open: bad block_count");
    uint32_t n_used = 8;
    if (qkg_kv_int(g, (arch + ".expert_used_count").c_str(), &v) == 0) n_used = (uint32_t)v;
    if (n_used < 1 || n_used > 16) return bad("qk_open: expert_used_count > 16 unsupported");
    if (qkg_kv_int(g, "tokenizer.ggml.eos_token_id", &v) == 0) eos = (uint32_t)v;
    if (qkg_kv_int(g, "tokenizer.ggml.bos_token_id", &v) == 0) bos = (uint32_t)v;
    layer_end = n_layer;
    // reference src/main.cpp:3594-3601: a:b selects a pipeline stage
    if (const char* lay = getenv("QK_LAYERS")) {
        unsigned a = 0, b = 0;
        if (sscanf(lay, "%u:%u", &a, &b) == 2 && a < b && b <= n_layer) { layer_first = a; layer_end = b; }
        else {
            if (err && err_len)
                snprintf(err, err_len, "qk_open: bad QK_LAYERS (want a:b with 0 <= a < b <= %u)", n_layer);
            return false;
        }
        if (split()) return bad("qk_open: QK_LAYERS pipeline stages are not part of this library (one GPU runs every layer)");
    }
    // Rows of one prefill pass.  Independent of QK_MAXB, which decides only WHICH positions are
    // prefilled at qk_slot_start (the reference's bookkeeping): more rows per pass read the weights
    // less often (40 layers: 6.7 k positions/s at 128, 8.7 k at 256, 11.3 k at 512, 12.7 k at 1024).
    if (const char* pr = getenv("QK_PREFILL_ROWS")) {
        const long x = atol(pr);
        if (x >= 16 && x <= 1024) pf_rows = (uint32_t)x;
        else fprintf(stderr, "QK_PREFILL_ROWS=%s out of range [16,1024]; using %u\n", pr, pf_rows);
    }
    if (const char* pc = getenv("QK_PCACHE")) { // reference src/main.cpp:4121-4125
        const long entries = strtol(pc, nullptr, 10);
        if (entries >= 1 && entries <= 256) n_state = (uint32_t)entries;
    }
    if (const char* mb = getenv("QK_MAXB")) { // reference src/main.cpp:3834-3838
        const long x = atol(mb);
        if (x >= 16 && x <= 1024) max_b = (uint32_t)x;
        else fprintf(stderr, "QK_MAXB=%s out of range [16,1024]; using %u\n", mb, max_b);
    }

    // reference src/main.cpp:3602-3609
    qkg_tensor t_embd, t_onorm, t_head;
    if (qkg_find(g, "token_embd.weight", &t_embd) || qkg_find(g, "output_norm.weight", &t_onorm) ||
        qkg_find(g, "output.weight", &t_head) || (t_embd.type != QKK_Q6_K && t_embd.type != QKK_Q8_0) ||
        t_head.type != QKK_Q6_K)
        return bad("qk_open: missing/unexpected embd/head tensors");
    // what the reference leaves to its shaders: shapes that fit each other
    if (t_embd.ne[0] != N_EMBD || t_head.ne[0] != N_EMBD || t_onorm.type != QKK_F32 || t_onorm.ne[0] != N_EMBD ||
        t_head.ne[1] < 1 || t_head.ne[1] > 0x7fffffffu || t_embd.ne[1] < t_head.ne[1] || t_embd.ne[1] > 0x7fffffffu ||
        !t_embd.nbytes || !t_head.nbytes || !t_onorm.nbytes)
        return bad("qk_open: missing/unexpected embd/head tensors");
    embd_type = (int)t_embd.type;
    embd_rows = (uint32_t)t_embd.ne[1];
    vocab = (uint32_t)t_head.ne[1];

    // the layers: MoE tensor sets (reference src/main.cpp:3611-3622, 1265-1311); with mixers (a
    // whole-model file: "ssm_a" marks a gated-DeltaNet layer, src/main.cpp:3919) or without any
    std::vector<qkg_moe_tensors> mt(n_layer);
    std::vector<qkg_tensor> pn(n_layer);
    std::vector<EngineLayer::Kind> kinds(n_layer, EngineLayer::MOE_ONLY);
    dn_kdiv = arch == "qwen3next" ? DN_HV / DN_HK : 0; // reference src/main.cpp:3588
    for (uint32_t l = 0; l < n_layer; l++) {
        char name[96];
        qkg_tensor tmp;
        snprintf(name, sizeof name, "blk.%u.ssm_a", l);
        if (qkg_find(g, name, &tmp) == 0) kinds[l] = EngineLayer::RECURRENT;
        snprintf(name, sizeof name, "blk.%u.attn_q.weight", l);
        if (kinds[l] == EngineLayer::MOE_ONLY && qkg_find(g, name, &tmp) == 0) kinds[l] = EngineLayer::ATTENTION;
        if (kinds[l] == EngineLayer::MOE_ONLY)
            for (const char* mixer : {"attn_qkv.weight", "attn_output.weight", "ssm_out.weight"}) {
                snprintf(name, sizeof name, "blk.%u.%s", l, mixer);
                if (qkg_find(g, name, &tmp) == 0) return bad("qk_open: a layer has mixer tensors but neither ssm_a nor attn_q");
            }
        if ((kinds[l] == EngineLayer::MOE_ONLY) != (kinds[0] == EngineLayer::MOE_ONLY))
            return bad("qk_open: layers with and without mixers in one file");
        if (qkg_moe_layer(g, l, &mt[l]) != 0) {
            if (err && err_len) snprintf(err, err_len, "qk_open: %s", qkk_last_error());
            return false;
        }
        if (l == 0 && (mt[0].n_expert < n_used || mt[0].n_expert > 512 || mt[0].n_ff % 256 != 0))
            return bad("qk_open: expert shape unsupported (n_expert <= 512, n_ff_exp % 256)");
        if (mt[l].n_embd != N_EMBD || mt[l].n_expert != mt[0].n_expert || mt[l].n_ff != mt[0].n_ff)
            return bad("qk_open: expert shape unsupported (n_embd 2048, uniform layers)");
        snprintf(name, sizeof name, "blk.%u.post_attention_norm.weight", l);
        if (qkg_find(g, name, &pn[l]) || pn[l].type != QKK_F32 || pn[l].ne[0] != N_EMBD || !pn[l].nbytes)
            return bad("qk_open: missing/unexpected post_attention_norm tensor");
    }

    // ---- device ----
    if (qk::require_device() != QKK_OK) return bad("qk_open: no HIP device: libqk.so has no CPU path");
    // Everything the open will hold on the device, before the first upload: the tensors of the file
    // (every one is uploaded at most once), per-slot state and the snapshot entries of the mixers, the
    // rows of a pass and the workspaces (a generous 64 KiB per row) -- a configuration that cannot fit
    // is refused here and not after gigabytes have been uploaded.
    uint64_t need = 64u << 20;
    for (uint64_t i = 0; i < qkg_n_tensors(g); i++) {
        qkg_tensor t;
        if (qkg_tensor_at(g, i, &t) == 0) need += t.nbytes + 512;
    }
    const bool with_mixers = kinds[0] != EngineLayer::MOE_ONLY;
    for (uint32_t l = 0; l < n_layer && with_mixers; l++) {
        const uint64_t per_slot = kinds[l] == EngineLayer::RECURRENT
                                      ? (uint64_t)DN_CH * 3 + (uint64_t)DN_HV * DN_DS * DN_DS
                                      : 2ull * FA_HKV * n_ctx * FA_DH;
        need += (n_slots + n_state) * per_slot * sizeof(float);
    }
    need += (uint64_t)(with_mixers ? pf_rows : MAX_ROWS) * (64u << 10) * sizeof(float) + (uint64_t)vocab * 80;
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return bad("qk_open: cannot query device memory");
    if (need > free_b) {
        if (err && err_len)
            snprintf(err, err_len, "qk_open: the model, %u slot(s) of state at n_ctx %u and the snapshots need about %.1f GB, "
                     "the device has %.1f GB free", n_slots, n_ctx, need / 1e9, free_b / 1e9);
        return false;
    }
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) return bad("qk_open: cannot create a stream");
    if (const char* sl = getenv("QK_WEIGHT_SLAB"); sl && atoi(sl) == 1) {
        uint64_t tensors = 0; // every tensor of the file at most once, each with its spare bytes and alignment
        for (uint64_t i = 0; i < qkg_n_tensors(g); i++) {
            qkg_tensor t;
            if (qkg_tensor_at(g, i, &t) == 0) tensors += t.nbytes + 512;
        }
        void* sp = nullptr;
        if (hipMalloc(&sp, tensors) != hipSuccess) { (void)hipGetLastError(); return bad("qk_open: device memory exhausted"); }
        dev_allocs.push_back(sp);
        slab = (uint8_t*)sp;
        slab_bytes = tensors;
    }

    const void* p = nullptr;
    if (!upload(t_embd, &d_embd, err, err_len) || !upload(t_head, &d_head, err, err_len) ||
        !upload(t_onorm, &p, err, err_len))
        return false;
    d_onorm = (const float*)p;
    layers.resize(n_layer);
    full_model = kinds[0] != EngineLayer::MOE_ONLY;
    for (uint32_t l = 0; l < n_layer; l++) {
        layers[l].kind = kinds[l];
        qkk_moe_layer& m = layers[l].moe;
        m.n_embd = mt[l].n_embd; m.n_ff = mt[l].n_ff; m.n_expert = mt[l].n_expert; m.n_used = mt[l].n_used;
        m.gu_type = mt[l].gu_type; m.down_type = mt[l].down_type;
        const void *gi = nullptr, *gis = nullptr;
        if (!upload(mt[l].gate_inp, &gi, err, err_len) || !upload(mt[l].gate_inp_shexp, &gis, err, err_len) ||
            !upload(mt[l].gate_exps, &m.gate_exps, err, err_len) || !upload(mt[l].up_exps, &m.up_exps, err, err_len) ||
            !upload(mt[l].down_exps, &m.down_exps, err, err_len) || !upload(mt[l].gate_shexp, &m.gate_shexp, err, err_len) ||
            !upload(mt[l].up_shexp, &m.up_shexp, err, err_len) || !upload(mt[l].down_shexp, &m.down_shexp, err, err_len) ||
            !upload(pn[l], &p, err, err_len))
            return false;
        m.gate_inp = (const float*)gi;
        m.gate_inp_shexp = (const float*)gis;
        layers[l].post_norm = (const float*)p;
    }

    cap = full_model ? pf_rows : MAX_ROWS;
    for (const EngineLayer& L : layers) ws_bytes = std::max(ws_bytes, qkk_moe_workspace_bytes(&L.moe, cap));
    hws_bytes = qkk_head_workspace_bytes(vocab, MAX_ROWS);
    if (!ws_bytes || !hws_bytes) return bad("qk_open: expert shape unsupported by the kernels");
    const size_t row_b = (size_t)cap * N_EMBD * sizeof(float);
    d_ids = (uint32_t*)dev_alloc(MAX_ROWS * 4, true);
    d_tok = (uint32_t*)dev_alloc(MAX_ROWS * 4, true);
    d_x = (float*)dev_alloc(row_b, true);
    d_xn[0] = (float*)dev_alloc(row_b, true);
    d_xn[1] = (float*)dev_alloc(row_b, true);
    d_last = (float*)dev_alloc(N_EMBD * sizeof(float), true);
    d_logits = (float*)dev_alloc((size_t)vocab * sizeof(float), true);
    d_sel = (qkk_sel*)dev_alloc(cap * sizeof(qkk_sel), true);
    d_ws = dev_alloc(ws_bytes, true);   // the kernels' workspaces start zero-filled
    d_hws = dev_alloc(hws_bytes, true);
    if (!d_ids || !d_tok || !d_x || !d_xn[0] || !d_xn[1] || !d_last || !d_logits || !d_sel || !d_ws || !d_hws)
        return bad("qk_open: device memory exhausted");
    if (hipHostMalloc((void**)&h_ids, MAX_ROWS * 4, hipHostMallocDefault) != hipSuccess ||
        hipHostMalloc((void**)&h_tok, MAX_ROWS * 4, hipHostMallocDefault) != hipSuccess ||
        hipHostMalloc((void**)&h_pos, MAX_ROWS * 4, hipHostMallocDefault) != hipSuccess)
        return bad("qk_open: cannot allocate pinned memory");
    memset(h_ids, 0, MAX_ROWS * 4);
    memset(h_tok, 0, MAX_ROWS * 4);
    memset(h_pos, 0, MAX_ROWS * 4);
    if (full_model && !load_mixers(g, err, err_len)) return false;
    cat_everywhere = full_model;
    qk::apply_env_options(qk::options()); // the QK_* switches as the environment holds them now
    dn_one_launch = qk::options().dn_fused && DN_HV == 2 * DN_HK;
    fused_norm = qk::options().fused_norm != 0;
    for (const EngineLayer& L : layers) cat_everywhere = cat_everywhere && L.cat.w != nullptr;
    if (hipDeviceSynchronize() != hipSuccess) return bad("qk_open: upload failed"); // fills and uploads are complete

    // One graph per dispatch depth z = highest active slot + 1 (the reference records one
    // command buffer per z, src/main.cpp:4169-4422).  Each depth runs once eagerly first, so
    // that whatever a launcher sets up on its first call is not part of a capture.
    prof_on = getenv("QK_STEP_PROF") != nullptr;
    counters_on = getenv("QK_COUNTERS") != nullptr;
    const bool use_graphs = !getenv("QK_NO_GRAPH");
    graphs.assign(use_graphs ? n_slots : 0, nullptr);
    for (uint32_t z = 1; z <= n_slots; z++) {
        if (run_rows(z, false) != 0) {
            if (err && err_len) snprintf(err, err_len, "qk_open: device step failed: %s", qkk_last_error());
            return false;
        }
        if (!use_graphs) continue;
        hipGraph_t graph = nullptr;
        if (hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) != hipSuccess)
            return bad("qk_open: graph capture failed");
        const int rc = copy_and_launch(z);
        const hipError_t ec = hipStreamEndCapture(st, &graph);
        if (rc != 0 || ec != hipSuccess || !graph) {
            if (graph) (void)hipGraphDestroy(graph);
            return bad("qk_open: graph capture failed");
        }
        const hipError_t ei = hipGraphInstantiate(&graphs[z - 1], graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (ei != hipSuccess) { graphs[z - 1] = nullptr; return bad("qk_open: graph instantiation failed"); }
    }
    if (full_model) // the warm-up steps above fed token 0 to every slot
        for (uint32_t sl = 0; sl < n_slots; sl++)
            if (reset_slot(sl) != 0) return bad("qk_open: device step failed");
    slots.assign(n_slots, Slot{});
    return true;
}

// reference src/main.cpp:4462-4646 with speculative decoding off: its phases 1 and 2 only move
// tokens a verify round left over, so phase 3 (serial steps) is the whole chunk.
int qk_engine::step_chunk(uint32_t* out_tok, uint32_t* out_cnt, uint32_t* out_fin)
{
    for (uint32_t s = 0; s < n_slots; s++) out_cnt[s] = 0;
    *out_fin = 0;
    int active_at_entry = 0;
    for (uint32_t s = 0; s < n_slots; s++)
        if (slots[s].active) active_at_entry++;
    if (!active_at_entry) return 0;

    auto finish = [&](uint32_t s) {
        slots[s].active = false;
        *out_fin |= 1u << s;
    };
    for (uint32_t step = 0; step < chunk; step++) {
        uint32_t n_act = 0, max_z = 0; // max_z: highest active slot + 1, the dispatch depth
        bool need = false;             // someone still owes prefill progress or emitted tokens
        for (uint32_t s = 0; s < n_slots; s++) {
            Slot& sl = slots[s];
            if (!sl.active) { h_ids[s] = 0; h_pos[s] = 0; continue; } // stepped with token 0 at position 0, like the reference
            n_act++;
            max_z = s + 1;
            if (sl.cursor < sl.prompt.size()) { // prefill: feed prompt[cursor] at position cursor
                h_ids[s] = sl.prompt[sl.cursor];
                h_pos[s] = sl.cursor;
                need = true;
            } else { // decode: feed the last sampled token at position pos
                h_ids[s] = sl.last;
                h_pos[s] = sl.pos;
                if (out_cnt[s] < chunk) need = true;
            }
        }
        if (!n_act || !need) break;
        // QK_STEP_PROF: the first pure decode step at depth 1 goes out kernel by kernel with an event behind each stage
        const bool profile = prof_on && !prof_printed && max_z == 1 && slots[0].active && slots[0].cursor >= slots[0].prompt.size();
        prof_armed = profile;
        const int rc_step = run_rows(max_z, !profile);
        prof_armed = false;
        if (rc_step) return rc_step;
        if (profile) {
            prof_report();
            prof_printed = true;
        }

        for (uint32_t s = 0; s < n_slots; s++) {
            Slot& sl = slots[s];
            if (!sl.active) continue;
            const uint32_t sampled = h_tok[s];
            const bool prefilling = sl.cursor < sl.prompt.size();
            if (prefilling && sl.cursor + 1 < sl.prompt.size()) {
                sl.cursor++; // still consuming the prompt: this step's logits are not used
                continue;
            }
            // this step produced a generated token (from the last prompt token, or a decode step)
            if (prefilling) { sl.cursor = (uint32_t)sl.prompt.size(); sl.pos = (uint32_t)sl.prompt.size(); }
            if (sampled == eos) { // not emitted
                if (!prefilling) sl.pos++;
                finish(s);
                continue;
            }
            if (out_cnt[s] < chunk) out_tok[s * chunk + out_cnt[s]++] = sampled; // one token per step: always fits
            sl.last = sampled;
            sl.gen++;
            if (!prefilling) sl.pos++;
            if (sl.pos >= n_ctx || sl.gen >= sl.max_gen) finish(s);
        }
    }
    return active_at_entry;
}

// reference src/main.cpp:5291-5307.  Only the unsplit engine exists here: tokens in, greedy ids
// out, no hidden rows on either side.  Rows are independent (no per-position state), so
// a chunk is cut into device steps of MAX_ROWS rows.
int qk_engine::stage_run(uint32_t slot, const uint32_t* toks, const float* hidden_in, uint32_t n, uint32_t base,
                         float* /*hidden_out*/, uint32_t* ids_out)
{
    if (slot >= n_slots || n < 1 || (uint64_t)base + n > n_ctx) return -1;
    if (!toks || hidden_in != nullptr) return -2;
    if (!ids_out) return -3;
    for (uint32_t i = 0; i < n; i++)
        if (toks[i] >= vocab) return -1;
    if (full_model) { // positions base .. base+n-1 of this slot, one after the other (the state is sequential)
        if (base == 0 && reset_slot(slot) != 0) return ERR_DEVICE; // base 0 starts from empty (reference src/main.cpp:4668-4675)
        if (int rc = prefill(slot, toks, n, base, ids_out)) return rc;
        last_run_rows = n; // the final position's normalised row is in d_last
        return 0;
    }
    for (uint32_t off = 0; off < n; off += MAX_ROWS) {
        const uint32_t rows = std::min(MAX_ROWS, n - off);
        memcpy(h_ids, toks + off, rows * sizeof(uint32_t));
        if (hipMemcpyAsync(d_ids, h_ids, rows * sizeof(uint32_t), hipMemcpyHostToDevice, st) != hipSuccess)
            return ERR_DEVICE;
        float* fin = nullptr;
        if (launch_rows(rows, &fin) != QKK_OK) return ERR_DEVICE;
        if (off + rows == n &&
            hipMemcpyAsync(d_last, fin + (size_t)(rows - 1) * N_EMBD, N_EMBD * sizeof(float), hipMemcpyDeviceToDevice,
                           st) != hipSuccess)
            return ERR_DEVICE;
        if (hipMemcpyAsync(h_tok, d_tok, rows * sizeof(uint32_t), hipMemcpyDeviceToHost, st) != hipSuccess ||
            hipStreamSynchronize(st) != hipSuccess)
            return ERR_DEVICE;
        memcpy(ids_out + off, h_tok, rows * sizeof(uint32_t));
    }
    last_run_rows = n;
    return 0;
}

// reference src/main.cpp:5309-5341: top-k (id, logit) of the final position of the last stage
// run, descending; equal logits in id order.
int qk_engine::stage_topk(uint32_t k, uint32_t* ids, float* vals)
{
    if (!ids || !vals || k < 1 || k > 256 || k > vocab) return -1;
    if (!last_run_rows) return -2;
    if (qkk_head_argmax(d_head, d_last, d_tok, d_logits, vocab, N_EMBD, 1, d_hws, hws_bytes, st) != QKK_OK)
        return ERR_DEVICE;
    std::vector<float> row(vocab);
    if (hipMemcpyAsync(row.data(), d_logits, (size_t)vocab * sizeof(float), hipMemcpyDeviceToHost, st) != hipSuccess ||
        hipStreamSynchronize(st) != hipSuccess)
        return ERR_DEVICE;
    std::vector<uint32_t> idx(vocab);
    for (uint32_t i = 0; i < vocab; i++) idx[i] = i;
    auto before = [&row](uint32_t a, uint32_t b) { return row[a] > row[b] || (row[a] == row[b] && a < b); };
    std::partial_sort(idx.begin(), idx.begin() + k, idx.end(), before);
    for (uint32_t i = 0; i < k; i++) {
        ids[i] = idx[i];
        vals[i] = row[idx[i]];
    }
    return 0;
}

extern "C" {

qk_engine* qk_open(const char* gguf_path, const qk_config* cfg, char* err, size_t err_len)
{
    if (!gguf_path || !cfg) { set_err(err, err_len, "qk_open: null arg"); return nullptr; }
    qk_engine* e = new (std::nothrow) qk_engine();
    if (!e) { set_err(err, err_len, "qk_open: oom"); return nullptr; }
    if (!e->open(gguf_path, *cfg, err, err_len)) { delete e; return nullptr; }
    return e;
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
uint32_t qk_n_embd(const qk_engine* e) { return e ? N_EMBD : 0; }

// reference src/main.cpp:5447-5516
int qk_slot_start(qk_engine* e, uint32_t slot, const uint32_t* prompt, uint32_t n_prompt, uint32_t max_gen,
                  uint32_t snap_prefix)
{
    if (!e || slot >= e->n_slots) return -1;
    if (e->split()) return -5;
    if (e->slots[slot].active) return -2;
    if (!prompt || n_prompt < 1 || (uint64_t)n_prompt + max_gen > e->n_ctx) return -3;
    for (uint32_t i = 0; i < n_prompt; i++)
        if (prompt[i] >= e->vocab) return -4;
    qk_engine::Slot& s = e->slots[slot];
    // Positions [0, n_prompt - 1) are batch-prefilled in chunks of max_b while 16 or more
    // remain, first up to the caller's history boundary, then up to the last prompt token; what
    // is left is consumed one token per serial step, and the last prompt token's step yields
    // the first generated token.  In a MoE-only model a prefilled position writes nothing (no
    // per-position state), so only the bookkeeping is left of the batch prefill.  The prefix
    // cache is not part of this library: start = 0.
    const uint32_t start = 0, target = n_prompt - 1;
    uint32_t done = start;
    auto batch_to = [&](uint32_t limit) {
        while (limit > done && limit - done >= 16) done += std::min(e->max_b, limit - done);
    };
    const uint32_t snap_at = (snap_prefix > start && snap_prefix < target) ? snap_prefix : 0;
    if (!getenv("QK_NO_BATCH")) {
        if (snap_at) batch_to(snap_at);
        batch_to(target);
    }
    if (e->full_model) {
        // a fresh request: clear the previous occupant's recurrent state, then the prefilled
        // positions on this slot alone (the last prompt token is left to the serial step as in the
        // reference)
        if (e->reset_slot(slot) != 0) return -6;
        if (done && e->prefill(slot, prompt, done, 0, nullptr) != 0) return -6;
    }
    s.cursor = done; s.pos = done;
    s.active = true;
    s.prompt.assign(prompt, prompt + n_prompt);
    s.gen = 0; s.max_gen = max_gen; s.last = 0;
    return 0;
}

void qk_slot_cancel(qk_engine* e, uint32_t slot)
{
    if (e && slot < e->n_slots) {
        e->slots[slot].active = false;
        e->slots[slot].prompt.clear();
    }
}

int qk_step_chunk(qk_engine* e, uint32_t* out_tokens, uint32_t* out_counts, uint32_t* out_finished)
{
    if (!e || !out_tokens || !out_counts || !out_finished) return -1;
    if (e->split()) return -5;
    return e->step_chunk(out_tokens, out_counts, out_finished);
}

int qk_stage_run(qk_engine* e, uint32_t slot, const uint32_t* toks, const float* hidden_in, uint32_t n, uint32_t base,
                 float* hidden_out, uint32_t* ids_out)
{
    if (!e) return -1;
    return e->stage_run(slot, toks, hidden_in, n, base, hidden_out, ids_out);
}

int qk_stage_topk(qk_engine* e, uint32_t k, uint32_t* ids, float* vals)
{
    if (!e) return -1;
    return e->stage_topk(k, ids, vals);
}

// reference src/main.cpp:5428-5445.  A MoE-only model has no per-position state: bounds only.
uint32_t qk_state_n(const qk_engine* e) { return e ? e->n_state : 0; }
int qk_state_save(qk_engine* e, uint32_t slot, uint32_t idx, uint32_t n_tok)
{
    if (!e || slot >= e->n_slots || idx >= e->n_state) return -1;
    return e->full_model ? e->copy_state(slot, idx, true, n_tok) : 0;
}
int qk_state_load(qk_engine* e, uint32_t slot, uint32_t idx, uint32_t n_tok)
{
    if (!e || slot >= e->n_slots || idx >= e->n_state) return -1;
    return e->full_model ? e->copy_state(slot, idx, false, n_tok) : 0;
}

} // extern "C"
