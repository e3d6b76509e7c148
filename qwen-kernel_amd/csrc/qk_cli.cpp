// qk_cli.cpp -- `qk`, the operator test program over libqk.so.
//
// The reference's `qk` binary runs its kernels on synthetic tensors from the command line
// (reference src/main.cpp:6952-6978): `qk suite`, `qk <format> [M] [K] [iters]`,
// `qk bgemm [M K N iters]`, `qk moe [layer] [iters]`, one line per case with microseconds per
// iteration, GB/s, GFLOP/s and the bytes moved (src/main.cpp:590-600), and a pass/fail verdict.
// This program has the same modes over the operator ABI of include/qk_kernels.h:
//
//   qk suite                          the five GEMV formats at 8192 x 8192, 200 iterations
//   qk f16|q8_0|q6_k|iq4_xs|iq3_xxs [M] [K] [iters]     defaults 16384 8192 100
//   qk bgemm [M] [K] [N] [iters]      the Q8_0 prefill GEMM, defaults 8192 2048 256 40
//   qk moe [seed] [iters] [slots] [experts]   one fused MoE layer (synthetic weights in place of a
//                                     model's layer index), defaults 0 200 1 256
//   qk head [batch] [iters]           the LM head 151936 x 2048 Q6_K with the argmax fused
// and, on the tensors of a model file named by QK_GGUF (reference src/main.cpp:846-915, 920-1254):
//   qk list [prefix]                  the file's tensors: name, type, dimensions
//   qk gguf <tensor> [iters]          y = W x on a named tensor (a 3-D tensor: its first slice, expert 0)
//   qk layer [layer] [iters] [slots]  the fused MoE step on the tensors blk.<layer>.ffn_* (the reference's
//                                     `qk moe [layer]`; `moe` here keeps its synthetic weights)
//   qk token <ids-file> <nGen> [tmax] [batch]   the whole model through the engine ABI of include/qk.h: the
//                                     prompt's ids from a file, nGen greedy tokens on `batch` slots fed the same
//                                     prompt (their streams must be identical), prefill and decode rates
//   qk warm <ids-file> <nGen> [tmax]  the same stream twice: after a prefill, and after restoring a snapshot of
//                                     the slot's state taken behind the prompt (reference src/main.cpp:2500-3062)
//
// The weights are seeded random valid blocks (every bit pattern of the quant fields is valid; the
// fp16 scales are |N(0,1)| * 1e-3), the activations N(0,1).  Iterations alternate over a ring of
// tensors larger than the 256 MB last-level cache, timed with HIP events on the launch stream.
// The verdict comes from a second computation on the device that shares no kernel with the first:
// the bit-exact dequantisation kernel followed by the dense fp32 GEMV (1e-3 of the largest output,
// the bar of the reference's own check, src/main.cpp:548-565); for `moe` the same rows through the
// expert-major matrix-core path.  No CPU arithmetic takes part.
#include <hip/hip_runtime.h>

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <string>
#include <vector>

#include "../../include/qk.h"
#include "../../include/qk_gguf.h"
#include "../../include/qk_kernels.h"

namespace {

constexpr double HBM_PEAK_GBPS = 8000.0, MFMA_F16_PEAK_TFLOPS = 2500.0;

#define HIP_OK(call)                                                                                        \
    do {                                                                                                    \
        const hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                             \
            fprintf(stderr, "qk: %s: %s\n", #call, hipGetErrorString(e_));                                  \
            exit(2);                                                                                        \
        }                                                                                                   \
    } while (0)
#define QK_OK(call)                                                                                         \
    do {                                                                                                    \
        const int rc_ = (call);                                                                             \
        if (rc_ != QKK_OK) {                                                                                \
            fprintf(stderr, "qk: %s: %d: %s\n", #call, rc_, qkk_last_error());                              \
            exit(2);                                                                                        \
        }                                                                                                   \
    } while (0)

// splitmix64: seeded, the same stream on every host
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {}
    uint64_t next()
    {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    float normal() // Box-Muller
    {
        const double u = std::max(uniform(), 1e-300), v = uniform();
        return (float)(sqrt(-2.0 * log(u)) * cos(6.283185307179586 * v));
    }
};

// float -> IEEE half bits, round to nearest even; values here are far inside the normal range
uint16_t half_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int32_t e = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
    uint32_t m = x & 0x7FFFFFu;
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        m |= 0x800000u;
        const int sh = 14 - e;
        uint32_t r = m >> sh;
        const uint32_t rem = m & ((1u << sh) - 1), halfway = 1u << (sh - 1);
        if (rem > halfway || (rem == halfway && (r & 1))) r++;
        return (uint16_t)(sign | r);
    }
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    uint32_t r = ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;
    return (uint16_t)(sign | r);
}

struct Format {
    const char* name;
    int type;
    uint32_t block_elems, block_bytes, scale_offset; // where the block's fp16 scale lies
};
const Format FORMATS[] = {{"f16", QKK_F16, 1, 2, 0},          {"q8_0", QKK_Q8_0, 32, 34, 0},     {"q6_k", QKK_Q6_K, 256, 210, 208},
                          {"iq4_xs", QKK_IQ4_XS, 256, 136, 0}, {"iq3_xxs", QKK_IQ3_XXS, 256, 98, 0}};

const Format* format_named(const char* n)
{
    for (const Format& f : FORMATS)
        if (!strcmp(f.name, n)) return &f;
    return nullptr;
}

// n_elems weights of a format as seeded random valid blocks
std::vector<uint8_t> random_tensor(const Format& f, uint64_t n_elems, uint64_t seed)
{
    Rng rng(seed);
    if (f.type == QKK_F16) {
        std::vector<uint8_t> out(n_elems * 2);
        uint16_t* h = (uint16_t*)out.data();
        for (uint64_t i = 0; i < n_elems; i++) h[i] = half_bits(rng.normal() * 0.05f);
        return out;
    }
    const uint64_t blocks = n_elems / f.block_elems;
    std::vector<uint8_t> out(blocks * f.block_bytes);
    uint64_t* w = (uint64_t*)out.data();
    for (uint64_t i = 0; i < out.size() / 8; i++) w[i] = rng.next();
    for (uint64_t i = out.size() / 8 * 8; i < out.size(); i++) out[i] = (uint8_t)rng.next();
    for (uint64_t b = 0; b < blocks; b++) {
        const uint16_t d = half_bits(fabsf(rng.normal()) * 1e-3f);
        memcpy(&out[b * f.block_bytes + f.scale_offset], &d, 2);
    }
    return out;
}

std::vector<float> random_rows(uint64_t n, uint64_t seed, float scale = 1.f)
{
    Rng rng(seed);
    std::vector<float> v(n);
    for (float& x : v) x = rng.normal() * scale;
    return v;
}

template <class T>
T* to_device(const std::vector<T>& h)
{
    T* d = nullptr;
    HIP_OK(hipMalloc((void**)&d, std::max<size_t>(h.size() * sizeof(T), 16)));
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}
template <class T>
T* device_zeros(size_t n)
{
    T* d = nullptr;
    HIP_OK(hipMalloc((void**)&d, std::max<size_t>(n * sizeof(T), 16)));
    HIP_OK(hipMemset(d, 0, std::max<size_t>(n * sizeof(T), 16)));
    return d;
}
std::vector<float> to_host(const float* d, size_t n)
{
    std::vector<float> h(n);
    HIP_OK(hipMemcpy(h.data(), d, n * 4, hipMemcpyDeviceToHost));
    return h;
}

// Microseconds per call of fn(i), i cycling over `ring`, by HIP events on `st` (one warm-up pass first).
template <class F>
double time_us(F fn, uint32_t iters, uint32_t ring, hipStream_t st)
{
    for (uint32_t i = 0; i < std::min(iters, ring); i++) fn(i % ring);
    hipEvent_t a, b;
    HIP_OK(hipEventCreate(&a));
    HIP_OK(hipEventCreate(&b));
    HIP_OK(hipStreamSynchronize(st));
    HIP_OK(hipEventRecord(a, st));
    for (uint32_t i = 0; i < iters; i++) fn(i % ring);
    HIP_OK(hipEventRecord(b, st));
    HIP_OK(hipEventSynchronize(b));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, a, b));
    HIP_OK(hipEventDestroy(a));
    HIP_OK(hipEventDestroy(b));
    return (double)ms * 1e3 / iters;
}

// max |a - b| / max |b|
double rel_maxabs(const std::vector<float>& a, const std::vector<float>& b)
{
    double top = 0, diff = 0;
    for (size_t i = 0; i < b.size(); i++) {
        top = std::max(top, (double)fabsf(b[i]));
        diff = std::max(diff, (double)fabsf(a[i] - b[i]));
    }
    return top > 0 ? diff / top : diff;
}

void print_line(double us, double bytes, double flops)
{
    // the reference's line (src/main.cpp:596-599) with the fraction of this device's HBM peak added
    printf("gpu: %8.1f us/iter | %7.1f GB/s (%4.1f%% of %.0f) | %8.1f GFLOP/s | %.1f MiB/iter\n", us, bytes / us / 1e3,
           bytes / us / 1e3 / HBM_PEAK_GBPS * 100, HBM_PEAK_GBPS, flops / us / 1e3, bytes / (1 << 20));
}

bool verdict(const char* what, double err, double bar)
{
    printf("check: %s: rel max-abs err %.3g (bar %.0e) -> %s\n", what, err, bar, err <= bar ? "OK" : "FAIL");
    return err <= bar;
}

// Second opinion on y = W x: bit-exact dequantisation, then the dense fp32 product (rows in pieces of at most 256 MiB)
bool check_gemv(int type, const uint8_t* W, const float* x, float* y, uint32_t M, uint32_t K, hipStream_t st)
{
    QK_OK(qkk_gemv(type, W, x, y, M, K, 1, st));
    const std::vector<float> got = to_host(y, M);
    std::vector<float> want(M);
    const uint32_t piece = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>(M, (64ull << 20) / K));
    float* dense = device_zeros<float>((size_t)piece * K);
    float* y2 = device_zeros<float>(piece);
    for (uint32_t r0 = 0; r0 < M; r0 += piece) {
        const uint32_t n = std::min(piece, M - r0);
        QK_OK(qkk_dequant(type, W + (size_t)r0 * qkk_row_bytes(type, K), dense, (uint64_t)n * K, st));
        QK_OK(qkk_gemv(QKK_F32, dense, x, y2, n, K, 1, st));
        HIP_OK(hipMemcpy(want.data() + r0, y2, (size_t)n * 4, hipMemcpyDeviceToHost));
    }
    HIP_OK(hipFree(dense)); HIP_OK(hipFree(y2));
    return verdict("against dequantise + dense fp32 product", rel_maxabs(got, want), 1e-3);
}

// y = W x for one format: ring of tensors, time, cross-check against dequantise + dense fp32 GEMV
bool case_gemv(const Format& f, uint32_t M, uint32_t K, uint32_t iters)
{
    if (qkk_row_bytes(f.type, K) == 0) {
        fprintf(stderr, "qk: K=%u is not a multiple of the %s block (%u)\n", K, f.name, f.block_elems);
        return false;
    }
    const size_t wbytes = (size_t)M * qkk_row_bytes(f.type, K);
    const uint32_t ring = (uint32_t)std::min<size_t>(64, std::max<size_t>(2, (320u << 20) / wbytes + 1));
    printf("== %s gemv M=%u K=%u iters=%u (ring of %u tensors, %.1f MiB each)\n", f.name, M, K, iters, ring,
           wbytes / 1048576.0);
    std::vector<uint8_t*> W(ring);
    for (uint32_t r = 0; r < ring; r++) W[r] = to_device(random_tensor(f, (uint64_t)M * K, 42 + r));
    float* x = to_device(random_rows(K, 43));
    float* y = device_zeros<float>(M);
    hipStream_t st = nullptr;
    const double us = time_us([&](uint32_t r) { QK_OK(qkk_gemv(f.type, W[r], x, y, M, K, 1, st)); }, iters, ring, st);
    print_line(us, (double)wbytes + 4.0 * K + 4.0 * M, 2.0 * M * K);
    const bool ok = check_gemv(f.type, W[0], x, y, M, K, st);
    for (uint8_t* p : W) HIP_OK(hipFree(p));
    HIP_OK(hipFree(x)); HIP_OK(hipFree(y));
    return ok;
}

// Y[N][M] = X[N][K] W[M][K]^T, W in Q8_0 (reference caseBGemm, src/main.cpp:5536-5672)
bool case_bgemm(uint32_t M, uint32_t K, uint32_t N, uint32_t iters)
{
    const Format& f = *format_named("q8_0");
    if (K % 32) {
        fprintf(stderr, "qk: K=%u is not a multiple of 32\n", K);
        return false;
    }
    const size_t wbytes = (size_t)M * qkk_row_bytes(QKK_Q8_0, K);
    const uint32_t ring = (uint32_t)std::min<size_t>(64, std::max<size_t>(2, (320u << 20) / wbytes + 1));
    printf("== q8_0 prefill gemm M=%u K=%u N=%u iters=%u (ring of %u)\n", M, K, N, iters, ring);
    std::vector<uint8_t*> W(ring);
    for (uint32_t r = 0; r < ring; r++) W[r] = to_device(random_tensor(f, (uint64_t)M * K, 42 + r));
    float* X = to_device(random_rows((size_t)N * K, 43));
    float* Y = device_zeros<float>((size_t)N * M);
    hipStream_t st = nullptr;
    const double us = time_us([&](uint32_t r) { QK_OK(qkk_gemm_q8_0(W[r], X, Y, M, K, N, st)); }, iters, ring, st);
    const double flops = 2.0 * M * K * N, bytes = (double)wbytes + 4.0 * N * K + 4.0 * N * M;
    print_line(us, bytes, flops);
    // the reference prints TFLOP/s against its matrix peak (src/main.cpp:5668-5672)
    printf("     %8.2f TFLOP/s = %.1f%% of the %.0f TFLOP/s dense fp16 matrix peak; %.0f tokens/s\n", flops / us / 1e6,
           flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS * 100, MFMA_F16_PEAK_TFLOPS, N / us * 1e6);
    QK_OK(qkk_gemm_q8_0(W[0], X, Y, M, K, N, st));
    const std::vector<float> got = to_host(Y, (size_t)N * M);
    // second opinion: one quantised GEMV per token (the one-row kernel, not the matrix cores)
    std::vector<float> want((size_t)N * M);
    float* y1 = device_zeros<float>(M);
    for (uint32_t n = 0; n < N; n++) {
        QK_OK(qkk_gemv(QKK_Q8_0, W[0], X + (size_t)n * K, y1, M, K, 1, st));
        HIP_OK(hipMemcpy(want.data() + (size_t)n * M, y1, (size_t)M * 4, hipMemcpyDeviceToHost));
    }
    const bool ok = verdict("against one GEMV per token", rel_maxabs(got, want), 1e-3);
    for (uint8_t* p : W) HIP_OK(hipFree(p));
    HIP_OK(hipFree(X)); HIP_OK(hipFree(Y)); HIP_OK(hipFree(y1));
    return ok;
}

struct Layer {
    qkk_moe_layer L;
    std::vector<void*> owned;
};

// One synthetic Qwen3-MoE layer at the reference model's shape (reference MoeT, src/main.cpp:1258-1311)
Layer make_layer(uint64_t seed, int down_type, uint32_t E)
{
    const uint32_t H = 2048, F = 512, k = 8;
    Layer out;
    auto up = [&](const std::vector<uint8_t>& h) { void* p = to_device(h); out.owned.push_back(p); return p; };
    const Format &iq3 = *format_named("iq3_xxs"), &q8 = *format_named("q8_0");
    const Format& dn = down_type == QKK_Q6_K ? *format_named("q6_k") : *format_named("iq4_xs");
    std::vector<float> gi = random_rows((size_t)E * H, seed * 16 + 1, 1.f / sqrtf((float)H)); // logits of order one
    std::vector<float> gis = random_rows(H, seed * 16 + 2, 1.f / sqrtf((float)H));
    float* d_gi = to_device(gi);
    float* d_gis = to_device(gis);
    out.owned.push_back(d_gi);
    out.owned.push_back(d_gis);
    out.L = qkk_moe_layer{H, F, E, k, QKK_IQ3_XXS, down_type, d_gi, d_gis,
                          up(random_tensor(iq3, (uint64_t)E * F * H, seed * 16 + 3)), up(random_tensor(iq3, (uint64_t)E * F * H, seed * 16 + 4)),
                          up(random_tensor(dn, (uint64_t)E * H * F, seed * 16 + 5)), up(random_tensor(q8, (uint64_t)F * H, seed * 16 + 6)),
                          up(random_tensor(q8, (uint64_t)F * H, seed * 16 + 7)), up(random_tensor(q8, (uint64_t)H * F, seed * 16 + 8))};
    return out;
}

// The fused step on a ring of layers of one shape: time, per stage, and the row-wise launches against the
// expert-major path (reference caseMoe, src/main.cpp:920-1254)
bool run_moe(std::vector<Layer>& layers, uint32_t iters, uint32_t slots, uint64_t seed)
{
    const qkk_moe_layer& L0 = layers[0].L;
    const uint32_t ring = (uint32_t)layers.size(), H = L0.n_embd, F = L0.n_ff, E = L0.n_expert, k = L0.n_used;
    float* X = to_device(random_rows((size_t)ring * slots * H, seed + 43));
    float* Y = device_zeros<float>((size_t)slots * H);
    qkk_sel* sel = device_zeros<qkk_sel>(slots);
    const size_t wsb = qkk_moe_workspace_bytes(&L0, std::max(slots, 16u));
    uint8_t* ws = device_zeros<uint8_t>(wsb);
    hipStream_t st = nullptr;
    auto step = [&](uint32_t r) { QK_OK(qkk_moe_decode(&layers[r].L, X + (size_t)r * slots * H, Y, sel, ws, wsb, slots, st)); };
    const double us = time_us(step, iters, ring, st);
    // bytes: router + shared gate row + shared expert + the distinct experts the rows picked (last step's picks)
    step(0);
    std::vector<qkk_sel> hs(slots);
    HIP_OK(hipMemcpy(hs.data(), sel, slots * sizeof(qkk_sel), hipMemcpyDeviceToHost));
    std::vector<uint32_t> ids;
    for (const qkk_sel& s : hs) ids.insert(ids.end(), s.ids, s.ids + k);
    std::sort(ids.begin(), ids.end());
    const size_t distinct = std::unique(ids.begin(), ids.end()) - ids.begin();
    const double per_expert = 2.0 * F * qkk_row_bytes(L0.gu_type, H) + (double)H * qkk_row_bytes(L0.down_type, F);
    const double bytes = (double)E * H * 4 + H * 4 + distinct * per_expert + 2.0 * F * qkk_row_bytes(QKK_Q8_0, H) +
                         (double)H * qkk_row_bytes(QKK_Q8_0, F) + slots * (2.0 * H * 4 + 160);
    print_line(us, bytes, slots * (2.0 * E * H + (k + 1) * 3 * 2.0 * F * H));
    printf("     %zu distinct experts; picks of row 0:", distinct);
    for (uint32_t i = 0; i < k; i++) printf(" %u(%.3f)", hs[0].ids[i], hs[0].w[i]);
    printf(" shared gate %.3f\n", hs[0].w_shared);
    // per stage, as the reference's QK_STEP_PROF does (src/main.cpp:4591-4632)
    for (uint32_t mask : {QKK_STAGE_ROUTE, QKK_STAGE_GATEUP, QKK_STAGE_DOWN}) {
        const double su = time_us([&](uint32_t r) {
            QK_OK(qkk_moe_decode_stages(&layers[r].L, X + (size_t)r * slots * H, Y, sel, ws, wsb, slots, mask, st)); }, iters, ring, st);
        printf("     stage %-7s %7.1f us\n", mask == QKK_STAGE_ROUTE ? "route" : mask == QKK_STAGE_GATEUP ? "gate/up" : "down", su);
    }
    // second opinion: the same rows, repeated to fill sixteen, through the expert-major matrix-core path
    step(0);
    const std::vector<float> got = to_host(Y, (size_t)slots * H);
    bool ok = true;
    if (slots > 10) printf("check: none (above ten rows both calls would take the expert-major path)\n");
    else if (H != 2048) printf("check: none (the expert-major path takes n_embd = 2048 only)\n");
    else {
        std::vector<float> x0 = to_host(X, (size_t)slots * H), x16((size_t)16 * H);
        for (uint32_t r = 0; r < 16; r++) memcpy(&x16[(size_t)r * H], &x0[(size_t)(r % slots) * H], H * 4);
        float* X16 = to_device(x16);
        float* Y16 = device_zeros<float>((size_t)16 * H);
        qkk_sel* sel16 = device_zeros<qkk_sel>(16);
        QK_OK(qkk_moe_decode(&L0, X16, Y16, sel16, ws, wsb, 16, st));
        std::vector<float> want = to_host(Y16, (size_t)slots * H);
        std::vector<qkk_sel> h16(16);
        HIP_OK(hipMemcpy(h16.data(), sel16, 16 * sizeof(qkk_sel), hipMemcpyDeviceToHost));
        bool same_ids = true;
        for (uint32_t r = 0; r < slots; r++) same_ids = same_ids && !memcmp(hs[r].ids, h16[r].ids, k * 4);
        printf("check: picks equal on both paths -> %s\n", same_ids ? "OK" : "FAIL");
        ok = verdict("row-wise launches against the expert-major path", rel_maxabs(got, want), 1e-3) && same_ids;
        HIP_OK(hipFree(X16)); HIP_OK(hipFree(Y16)); HIP_OK(hipFree(sel16));
    }
    for (Layer& l : layers)
        for (void* p : l.owned) HIP_OK(hipFree(p));
    HIP_OK(hipFree(X)); HIP_OK(hipFree(Y)); HIP_OK(hipFree(sel)); HIP_OK(hipFree(ws));
    return ok;
}

bool case_moe(uint32_t seed, uint32_t iters, uint32_t slots, uint32_t E)
{
    if (slots < 1 || slots > 4096 || E < 8 || E > QKK_MAX_EXPERTS) {
        fprintf(stderr, "qk: slots %u outside 1..4096 or experts %u outside 8..%u\n", slots, E, QKK_MAX_EXPERTS);
        return false;
    }
    const uint32_t ring = 4;
    const int down = slots == 1 ? QKK_IQ4_XS : QKK_Q6_K; // the reference's 35B model mixes both down types
    printf("== fused moe layer (synthetic, seed %u): %u experts, %u slot(s), down %s, iters=%u, ring of %u layers\n", seed, E,
           slots, down == QKK_Q6_K ? "q6_k" : "iq4_xs", iters, ring);
    std::vector<Layer> layers;
    for (uint32_t r = 0; r < ring; r++) layers.push_back(make_layer(seed * 8 + r, down, E));
    return run_moe(layers, iters, slots, seed);
}

// ---- the tensors of a model file ----------------------------------------------------------------

const char* type_name(uint32_t t)
{
    switch (t) {
    case QKK_F32: return "f32";
    case QKK_F16: return "f16";
    case QKK_Q8_0: return "q8_0";
    case QKK_Q6_K: return "q6_k";
    case QKK_IQ4_XS: return "iq4_xs";
    case QKK_IQ3_XXS: return "iq3_xxs";
    default: return "other";
    }
}

// The model file: QK_GGUF, as in the reference (src/main.cpp:846-856: no compiled-in default)
qkg_file* open_model()
{
    const char* path = getenv("QK_GGUF");
    if (!path || !*path) {
        fprintf(stderr, "qk: no model path. Set QK_GGUF=/path/to/model.gguf\n");
        exit(1);
    }
    qkg_file* f = qkg_open(path);
    if (!f) {
        fprintf(stderr, "qk: %s: %s\n", path, qkk_last_error());
        exit(1);
    }
    return f;
}

bool case_list(const char* prefix)
{
    qkg_file* f = open_model();
    printf("gguf v%u, %u shard(s), %llu tensors\n", qkg_version(f), qkg_n_shards(f), (unsigned long long)qkg_n_tensors(f));
    for (uint64_t i = 0; i < qkg_n_tensors(f); i++) {
        qkg_tensor t;
        if (qkg_tensor_at(f, i, &t) != QKK_OK) continue;
        if (prefix && strncmp(t.name, prefix, strlen(prefix))) continue;
        printf("%-40s %-8s [%llu, %llu, %llu, %llu] %.1f MiB\n", t.name, type_name(t.type), (unsigned long long)t.ne[0],
               (unsigned long long)t.ne[1], (unsigned long long)t.ne[2], (unsigned long long)t.ne[3], t.nbytes / 1048576.0);
    }
    qkg_close(f);
    return true;
}

// y = W x on a tensor of the file (reference caseGguf, src/main.cpp:858-915)
bool case_gguf(const char* name, uint32_t iters)
{
    qkg_file* f = open_model();
    qkg_tensor t;
    if (qkg_find(f, name, &t) != QKK_OK) {
        fprintf(stderr, "qk: tensor '%s' not found (try: qk list)\n", name);
        qkg_close(f);
        return false;
    }
    const uint32_t K = (uint32_t)t.ne[0], M = (uint32_t)t.ne[1];
    const size_t row = qkk_row_bytes((int)t.type, K);
    printf("== gguf %s  %s  ne=[%llu,%llu,%llu]\n", name, type_name(t.type), (unsigned long long)t.ne[0],
           (unsigned long long)t.ne[1], (unsigned long long)t.ne[2]);
    if (!row || t.n_dims < 2) {
        fprintf(stderr, "qk: no kernel for a %u-dimensional tensor of type %s\n", t.n_dims, type_name(t.type));
        qkg_close(f);
        return false;
    }
    if (t.ne[2] > 1) printf("3-D tensor: its first slice (expert 0)\n");
    const size_t wbytes = (size_t)M * row;
    printf("gemv M=%u K=%u, W %.1f MiB\n", M, K, wbytes / 1048576.0);
    uint8_t* W = nullptr;
    HIP_OK(hipMalloc((void**)&W, std::max<size_t>(wbytes, 16)));
    HIP_OK(hipMemcpy(W, t.data, wbytes, hipMemcpyHostToDevice));
    qkg_close(f);
    float* x = to_device(random_rows(K, 43));
    float* y = device_zeros<float>(M);
    hipStream_t st = nullptr;
    const double us = time_us([&](uint32_t) { QK_OK(qkk_gemv((int)t.type, W, x, y, M, K, 1, st)); }, iters, 1, st);
    print_line(us, (double)wbytes + 4.0 * K + 4.0 * M, 2.0 * M * K);
    bool ok = true;
    if (t.type == QKK_F32) printf("check: none (the dense fp32 product is the second opinion of the others)\n");
    else ok = check_gemv((int)t.type, W, x, y, M, K, st);
    HIP_OK(hipFree(W)); HIP_OK(hipFree(x)); HIP_OK(hipFree(y));
    return ok;
}

// The fused MoE step on the tensors of one layer of the file (reference caseMoe, src/main.cpp:920-1254)
bool case_layer(uint32_t layer, uint32_t iters, uint32_t slots)
{
    if (slots < 1 || slots > 4096) {
        fprintf(stderr, "qk: slots %u outside 1..4096\n", slots);
        return false;
    }
    qkg_file* f = open_model();
    qkg_moe_tensors mt;
    if (qkg_moe_layer(f, layer, &mt) != QKK_OK) {
        fprintf(stderr, "qk: layer %u: %s\n", layer, qkk_last_error());
        qkg_close(f);
        return false;
    }
    printf("== fused moe layer blk.%u: n_embd %u, n_ff %u, %u experts, %u used, down %s, %u slot(s), iters=%u\n", layer, mt.n_embd,
           mt.n_ff, mt.n_expert, mt.n_used, type_name((uint32_t)mt.down_type), slots, iters);
    std::vector<Layer> layers(1);
    Layer& out = layers[0];
    auto up = [&](const qkg_tensor& t) {
        void* p = nullptr;
        HIP_OK(hipMalloc(&p, std::max<size_t>(t.nbytes, 16)));
        HIP_OK(hipMemcpy(p, t.data, t.nbytes, hipMemcpyHostToDevice));
        out.owned.push_back(p);
        return p;
    };
    out.L = qkk_moe_layer{mt.n_embd, mt.n_ff, mt.n_expert, mt.n_used, mt.gu_type, mt.down_type,
                          (const float*)up(mt.gate_inp), (const float*)up(mt.gate_inp_shexp), up(mt.gate_exps), up(mt.up_exps),
                          up(mt.down_exps), up(mt.gate_shexp), up(mt.up_shexp), up(mt.down_shexp)};
    qkg_close(f);
    return run_moe(layers, iters, slots, layer);
}

bool case_head(uint32_t batch, uint32_t iters)
{
    const uint32_t V = 151936, K = 2048, ring = 2;
    if (batch < 1 || batch > 16) {
        fprintf(stderr, "qk: batch %u outside 1..16\n", batch);
        return false;
    }
    const Format& f = *format_named("q6_k");
    printf("== lm head + argmax: q6_k %u x %u, batch %u, iters=%u\n", V, K, batch, iters);
    uint8_t* W[ring];
    for (uint32_t r = 0; r < ring; r++) W[r] = to_device(random_tensor(f, (uint64_t)V * K, 77 + r));
    float* X = to_device(random_rows((size_t)batch * K, 43));
    uint32_t* tok = device_zeros<uint32_t>(batch);
    float* logits = device_zeros<float>((size_t)batch * V);
    const size_t wsb = qkk_head_workspace_bytes(V, batch);
    uint8_t* ws = device_zeros<uint8_t>(wsb);
    hipStream_t st = nullptr;
    const double us = time_us([&](uint32_t r) { QK_OK(qkk_head_argmax(W[r], X, tok, nullptr, V, K, batch, ws, wsb, st)); }, iters, ring, st);
    print_line(us, (double)V * qkk_row_bytes(QKK_Q6_K, K) + batch * (4.0 * K + 4), 2.0 * V * K * batch);
    // second opinion: the logits written out, the two-pass argmax over them
    QK_OK(qkk_head_argmax(W[0], X, tok, logits, V, K, batch, ws, wsb, st));
    uint32_t* tok2 = device_zeros<uint32_t>(batch);
    QK_OK(qkk_argmax(logits, tok2, V, batch, st));
    std::vector<uint32_t> a(batch), b(batch);
    HIP_OK(hipMemcpy(a.data(), tok, batch * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(b.data(), tok2, batch * 4, hipMemcpyDeviceToHost));
    const bool ok = a == b;
    printf("check: fused argmax equals the argmax of the written logits (row 0: %u) -> %s\n", a[0], ok ? "OK" : "FAIL");
    for (uint8_t* p : W) HIP_OK(hipFree(p));
    HIP_OK(hipFree(X)); HIP_OK(hipFree(tok)); HIP_OK(hipFree(tok2)); HIP_OK(hipFree(logits)); HIP_OK(hipFree(ws));
    return ok;
}

// ---- the whole model through the engine ABI ---------------------------------------------------

double ms_since(std::chrono::steady_clock::time_point t0)
{
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

// ids separated by commas, blanks or newlines (reference src/main.cpp:2502-2509)
bool read_ids(const char* path, std::vector<uint32_t>& out)
{
    FILE* f = fopen(path, "r");
    if (!f) {
        perror(path);
        return false;
    }
    long v;
    while (fscanf(f, "%ld%*[, \n\r\t]", &v) == 1) out.push_back((uint32_t)std::max(0l, v));
    fclose(f);
    return true;
}

qk_engine* open_engine(uint32_t slots, uint32_t tmax)
{
    const char* path = getenv("QK_GGUF");
    if (!path || !*path) {
        fprintf(stderr, "qk: no model path. Set QK_GGUF=/path/to/model.gguf\n");
        exit(1);
    }
    const qk_config cfg{slots, std::max(64u, tmax), 8};
    char err[512] = "";
    qk_engine* e = qk_open(path, &cfg, err, sizeof err);
    if (!e) {
        fprintf(stderr, "qk: %s: %s\n", path, err);
        exit(1);
    }
    return e;
}

// reference caseToken (src/main.cpp:2500-3062): prefill, nGen greedy steps on nB identical streams
bool case_token(const char* ids_file, uint32_t n_gen, uint32_t tmax, uint32_t nb)
{
    std::vector<uint32_t> prompt;
    if (!read_ids(ids_file, prompt)) return false;
    if (prompt.empty() || n_gen == 0 || prompt.size() + n_gen > tmax) {
        fprintf(stderr, "qk: bad prompt (%zu ids, %u to generate, tmax %u)\n", prompt.size(), n_gen, tmax);
        return false;
    }
    if (nb < 1 || nb > 16) {
        fprintf(stderr, "qk: batch must be 1..16\n");
        return false;
    }
    qk_engine* e = open_engine(nb, tmax);
    const uint32_t chunk = qk_chunk(e);
    printf("token mode: %zu prompt ids, gen %u, vocab %u, tmax %u, batch %u\n", prompt.size(), n_gen, qk_n_vocab(e), tmax, nb);
    auto t0 = std::chrono::steady_clock::now();
    for (uint32_t s = 0; s < nb; s++) {
        const int rc = qk_slot_start(e, s, prompt.data(), (uint32_t)prompt.size(), n_gen, 0);
        if (rc != 0) {
            fprintf(stderr, "qk: qk_slot_start(slot %u) returned %d\n", s, rc);
            qk_close(e);
            return false;
        }
    }
    const double prefill_ms = ms_since(t0);
    printf("prefill: %zu tokens x %u streams in %.1f ms (%.2f ms/token)\n", prompt.size(), nb, prefill_ms,
           prefill_ms / (prompt.size() * nb));
    std::vector<std::vector<uint32_t>> gen(nb);
    std::vector<uint32_t> toks((size_t)nb * chunk), counts(nb);
    uint32_t finished = 0, calls = 0;
    t0 = std::chrono::steady_clock::now();
    for (;;) {
        const int active = qk_step_chunk(e, toks.data(), counts.data(), &finished);
        if (active < 0) {
            fprintf(stderr, "qk: qk_step_chunk returned %d\n", active);
            qk_close(e);
            return false;
        }
        if (active == 0) break;
        calls++;
        for (uint32_t s = 0; s < nb; s++) gen[s].insert(gen[s].end(), &toks[(size_t)s * chunk], &toks[(size_t)s * chunk] + counts[s]);
    }
    const double gen_ms = ms_since(t0);
    const size_t n0 = gen[0].size();
    bool same = true;
    for (uint32_t s = 1; s < nb; s++) same = same && gen[s] == gen[0];
    printf("decode: %zu tokens x %u streams in %.1f ms (%u calls of %u steps) -> %.2f ms/step | per-stream %.1f tok/s | aggregate %.1f tok/s\n",
           n0, nb, gen_ms, calls, chunk, n0 ? gen_ms / n0 : 0.0, n0 * 1000.0 / gen_ms, (double)n0 * nb * 1000.0 / gen_ms);
    if (n0 < n_gen) printf("the stream ended at the end-of-sequence token %u after %zu tokens\n", qk_eos_token(e), n0);
    if (nb > 1) printf("streams identical: %s\n", same ? "YES" : "NO");
    printf("GEN:");
    for (uint32_t id : gen[0]) printf(" %u", id);
    printf("\n");
    qk_close(e);
    return same;
}

// reference caseToken with warmDemo (src/main.cpp:2975-3050): the cost of a cached prefix against a prefill
bool case_warm(const char* ids_file, uint32_t n_gen, uint32_t tmax)
{
    std::vector<uint32_t> prompt;
    if (!read_ids(ids_file, prompt)) return false;
    if (prompt.empty() || n_gen == 0 || prompt.size() + n_gen > tmax) {
        fprintf(stderr, "qk: bad prompt (%zu ids, %u to generate, tmax %u)\n", prompt.size(), n_gen, tmax);
        return false;
    }
    qk_engine* e = open_engine(1, tmax);
    const uint32_t n = (uint32_t)prompt.size();
    if (qk_state_n(e) == 0) {
        fprintf(stderr, "qk: the engine keeps no state snapshots\n");
        qk_close(e);
        return false;
    }
    printf("warm mode: %u prompt ids, gen %u, tmax %u, %u snapshot entries\n", n, n_gen, tmax, qk_state_n(e));
    std::vector<uint32_t> ids(n);
    auto t0 = std::chrono::steady_clock::now();
    int rc = qk_stage_run(e, 0, prompt.data(), nullptr, n, 0, nullptr, ids.data());
    const double prefill_ms = ms_since(t0);
    if (rc != 0) {
        fprintf(stderr, "qk: qk_stage_run returned %d\n", rc);
        qk_close(e);
        return false;
    }
    const uint32_t first = ids[n - 1]; // the token behind the prompt: kept with the snapshot, as the reference keeps its logits
    t0 = std::chrono::steady_clock::now();
    rc = qk_state_save(e, 0, 0, n);
    const double snap_ms = ms_since(t0);
    auto decode = [&](std::vector<uint32_t>& out, double& ms) {
        out.assign(1, first);
        const auto t1 = std::chrono::steady_clock::now();
        for (uint32_t i = 1; i < n_gen && rc == 0; i++) {
            uint32_t next = 0;
            rc = qk_stage_run(e, 0, &out.back(), nullptr, 1, n + i - 1, nullptr, &next);
            out.push_back(next);
        }
        ms = ms_since(t1);
    };
    std::vector<uint32_t> cold, warm;
    double cold_ms = 0, warm_ms = 0;
    if (rc == 0) decode(cold, cold_ms);
    t0 = std::chrono::steady_clock::now();
    if (rc == 0) rc = qk_state_load(e, 0, 0, n); // a "new request" with the same prefix
    const double restore_ms = ms_since(t0);
    if (rc == 0) decode(warm, warm_ms);
    if (rc != 0) {
        fprintf(stderr, "qk: a state or stage call returned %d\n", rc);
        qk_close(e);
        return false;
    }
    const bool eq = warm == cold;
    printf("cold start: prefill %u tokens = %.1f ms before the first token\n", n, prefill_ms);
    printf("warm start: restore the snapshot = %.1f ms before the first token (snapshot %.1f ms, paid once)\n", restore_ms, snap_ms);
    printf("decode: cold %.1f ms, warm %.1f ms for %u tokens; warm stream identical to cold: %s\n", cold_ms, warm_ms, n_gen,
           eq ? "YES" : "NO");
    printf("GEN:");
    for (uint32_t id : cold) printf(" %u", id);
    printf("\n");
    if (!eq) {
        printf("WARM:");
        for (uint32_t id : warm) printf(" %u", id);
        printf("\n");
    }
    qk_close(e);
    return eq;
}

void usage()
{
    fprintf(stderr, "usage: qk suite\n"
                    "       qk f16|q8_0|q6_k|iq4_xs|iq3_xxs [M] [K] [iters]\n"
                    "       qk bgemm [M] [K] [N] [iters]\n"
                    "       qk moe [seed] [iters] [slots] [experts]\n"
                    "       qk head [batch] [iters]\n"
                    "       QK_GGUF=model.gguf qk list [prefix] | gguf <tensor> [iters] | layer [layer] [iters] [slots]\n"
                    "       QK_GGUF=model.gguf qk token <ids-file> <nGen> [tmax] [batch] | warm <ids-file> <nGen> [tmax]\n");
}

} // namespace

int main(int argc, char** argv)
{
    if (argc < 2) {
        usage();
        return 1;
    }
    const std::string mode = argv[1];
    auto arg_u = [&](int i, uint32_t dflt) { return argc > i ? (uint32_t)strtoul(argv[i], nullptr, 10) : dflt; };
    const bool known = mode == "suite" || mode == "bgemm" || mode == "moe" || mode == "head" || mode == "list" || mode == "gguf" ||
                       mode == "layer" || mode == "token" || mode == "warm" || format_named(mode.c_str());
    if (!known || (mode == "gguf" && argc < 3) || ((mode == "token" || mode == "warm") && argc < 4)) {
        usage();
        return 1;
    }
    if (mode == "list") return case_list(argc > 2 ? argv[2] : nullptr) ? 0 : 1; // host only
    char arch[64] = "";
    uint32_t cus = 0;
    if (qkk_device_info(arch, sizeof arch, &cus) < 1) {
        fprintf(stderr, "qk: no HIP device: libqk.so has no CPU path\n");
        return 2;
    }
    printf("device: %s, %u CUs\n", arch, cus);
    bool ok = true;
    if (mode == "suite") {
        for (const Format& f : FORMATS) ok &= case_gemv(f, 8192, 8192, 200);
    } else if (mode == "bgemm") {
        ok = case_bgemm(arg_u(2, 8192), arg_u(3, 2048), arg_u(4, 256), arg_u(5, 40));
    } else if (mode == "moe") {
        ok = case_moe(arg_u(2, 0), arg_u(3, 200), arg_u(4, 1), arg_u(5, 256));
    } else if (mode == "head") {
        ok = case_head(arg_u(2, 1), arg_u(3, 40));
    } else if (mode == "gguf") {
        ok = case_gguf(argv[2], arg_u(3, 100));
    } else if (mode == "layer") {
        ok = case_layer(arg_u(2, 0), arg_u(3, 200), arg_u(4, 1));
    } else if (mode == "token") {
        ok = case_token(argv[2], arg_u(3, 12), arg_u(4, 128), arg_u(5, 1));
    } else if (mode == "warm") {
        ok = case_warm(argv[2], arg_u(3, 12), arg_u(4, 128));
    } else {
        ok = case_gemv(*format_named(mode.c_str()), arg_u(2, 16384), arg_u(3, 8192), arg_u(4, 100));
    }
    printf("%s\n", ok ? "ALL OK" : "FAILED");
    return ok ? 0 : 1;
}
