// qk_head.hip -- LM head (Q6_K GEMV) with greedy sampling fused into the epilogue, and the
// stand-alone argmax.
//
// Each wave keeps the best (logit, id) of the rows it produced; a block folds its waves,
// writes one candidate, and the block that finishes last folds all candidates into the
// token id.  Ties go to the lower id; a logit must beat -3.4e38 to be chosen
// (reference shaders/argmax1.comp:25-33, argmax2.comp:20-28).
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {

constexpr float ARG_FLOOR = -3.4e38f;

__device__ __forceinline__ bool better(float v, uint32_t i, float bv, uint32_t bi)
{
    return v > bv || (v == bv && i < bi);
}

struct HeadWs {
    uint32_t* counter; // [batch]
    float* cand_v;     // [batch][blocks]
    uint32_t* cand_i;  // [batch][blocks]
};

// Folds n candidates with one block of 256 threads; thread 0 returns the winner.
__device__ static uint32_t fold_candidates(const volatile float* cv, const volatile uint32_t* ci,
                                           uint32_t n, float* s_v, uint32_t* s_i)
{
    float bv = ARG_FLOOR;
    uint32_t bi = 0xFFFFFFFFu;
    for (uint32_t c = threadIdx.x; c < n; c += 256) {
        const float v = cv[c];
        const uint32_t i = ci[c];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    s_v[threadIdx.x] = bv;
    s_i[threadIdx.x] = bi;
    __syncthreads();
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s && better(s_v[threadIdx.x + s], s_i[threadIdx.x + s], s_v[threadIdx.x], s_i[threadIdx.x])) {
            s_v[threadIdx.x] = s_v[threadIdx.x + s];
            s_i[threadIdx.x] = s_i[threadIdx.x + s];
        }
        __syncthreads();
    }
    return s_i[0] == 0xFFFFFFFFu ? 0u : s_i[0];
}

template <int PASSES, int RIF>
__global__ __launch_bounds__(256) void head_q6k_kernel(const uint8_t* __restrict__ W,
                                                       const float* __restrict__ X,
                                                       float* __restrict__ logits_out,
                                                       uint32_t* __restrict__ tok, HeadWs ws, uint32_t V,
                                                       uint32_t K, uint32_t row_bytes)
{
    __shared__ float s_v[256];
    __shared__ uint32_t s_i[256];
    __shared__ uint32_t s_last;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t b = blockIdx.y;
    const float* x = X + (size_t)b * K;

    XSlice xs[PASSES];
    float xsum[PASSES][4];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        load_xslice<QKK_Q6_K>(xs[p], x + p * 2048, lane);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) s += xs[p].v[c * 8 + i];
            xsum[p][c] = s;
        }
    }
    const uint32_t pass_bytes = row_bytes / PASSES;
    float bv = ARG_FLOOR;
    uint32_t bi = 0xFFFFFFFFu;
    // chunks of RIF rows dealt round-robin to the waves; a wave's rows ascend
    for (uint32_t r0 = (blockIdx.x * 4 + wave) * RIF; r0 < V; r0 += gridDim.x * 4 * RIF) {
        LaneW<QKK_Q6_K> w[RIF][PASSES];
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            const uint32_t r = min(r0 + i, V - 1);
#pragma unroll
            for (int p = 0; p < PASSES; p++)
                w[i][p].load(W + (size_t)r * row_bytes + (size_t)p * pass_bytes, lane);
        }
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) acc += w[i][p].dot(xs[p], xsum[p], nullptr, lane);
            acc = wave_sum(acc);
            const uint32_t r = r0 + i;
            if (r < V) {
                if (logits_out && lane == 0) logits_out[(size_t)b * V + r] = acc;
                if (acc > bv) { bv = acc; bi = r; } // rows ascend: strict '>' keeps the lowest id
            }
        }
    }

    // fold the four waves of the block
    if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 4; wv++)
            if (better(s_v[wv], s_i[wv], bv, bi)) { bv = s_v[wv]; bi = s_i[wv]; }
        ws.cand_v[(size_t)b * gridDim.x + blockIdx.x] = bv;
        ws.cand_i[(size_t)b * gridDim.x + blockIdx.x] = bi;
        __threadfence();
        s_last = atomicAdd(&ws.counter[b], 1u) == gridDim.x - 1 ? 1u : 0u;
    }
    __syncthreads();
    if (s_last) {
        __threadfence();
        const uint32_t t = fold_candidates(ws.cand_v + (size_t)b * gridDim.x, ws.cand_i + (size_t)b * gridDim.x,
                                           gridDim.x, s_v, s_i);
        if (threadIdx.x == 0) {
            tok[b] = t;
            ws.counter[b] = 0u;
        }
    }
}

// One block per row; ties to the lower index.
__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ logits,
                                                     uint32_t* __restrict__ tok, uint32_t n)
{
    __shared__ float s_v[256];
    __shared__ uint32_t s_i[256];
    const float* row = logits + (size_t)blockIdx.x * n;
    float bv = ARG_FLOOR;
    uint32_t bi = 0xFFFFFFFFu;
    for (uint32_t i = threadIdx.x; i < n; i += 256) {
        const float v = row[i];
        if (v > bv) { bv = v; bi = i; }
    }
    s_v[threadIdx.x] = bv;
    s_i[threadIdx.x] = bi;
    __syncthreads();
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s && better(s_v[threadIdx.x + s], s_i[threadIdx.x + s], s_v[threadIdx.x], s_i[threadIdx.x])) {
            s_v[threadIdx.x] = s_v[threadIdx.x + s];
            s_i[threadIdx.x] = s_i[threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) tok[blockIdx.x] = s_i[0] == 0xFFFFFFFFu ? 0u : s_i[0];
}

static uint32_t head_blocks(uint32_t V, uint32_t rif)
{
    const uint32_t waves = (V + rif - 1) / rif;
    return std::min((waves + 3) / 4, persistent_blocks());
}
constexpr uint32_t HEAD_RIF = 4;

} // namespace qk

using namespace qk;

extern "C" {

size_t qkk_head_workspace_bytes(uint32_t V, uint32_t batch)
{
    if (V == 0 || batch == 0) return 0;
    const size_t blocks = head_blocks(V, 1); // upper bound over the kernels' RIF choices
    return 256 + (size_t)batch * blocks * 8;
}

int qkk_head_argmax(const void* W, const float* X, uint32_t* tok, float* logits, uint32_t V, uint32_t K,
                    uint32_t batch, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!W || !X || !tok || !workspace) return fail(QKK_EINVAL, "qkk_head_argmax: null pointer");
    if (V == 0 || batch == 0) return fail(QKK_EINVAL, "qkk_head_argmax: V and batch must be positive");
    if (batch > 64) return fail(QKK_ESHAPE, "qkk_head_argmax: batch %u exceeds 64", batch);
    if (K != 2048 && K != 4096) return fail(QKK_ESHAPE, "qkk_head_argmax: K=%u not supported (2048 or 4096)", K);
    if (!aligned16(W) || !aligned16(X) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return fail(QKK_EINVAL, "qkk_head_argmax: W/X must be 16-byte and workspace 256-byte aligned");
    if (workspace_bytes < qkk_head_workspace_bytes(V, batch))
        return fail(QKK_EWORKSPACE, "qkk_head_argmax: workspace %zu < %zu bytes", workspace_bytes,
                    qkk_head_workspace_bytes(V, batch));
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    const uint32_t rif = K == 2048 ? HEAD_RIF : 2;
    const uint32_t blocks = head_blocks(V, rif);
    HeadWs ws;
    ws.counter = (uint32_t*)workspace;
    ws.cand_v = (float*)((uint8_t*)workspace + 256);
    ws.cand_i = (uint32_t*)(ws.cand_v + (size_t)batch * blocks);
    const uint32_t rb = (uint32_t)qkk_row_bytes(QKK_Q6_K, K);
    if (K == 2048)
        hipLaunchKernelGGL((head_q6k_kernel<1, HEAD_RIF>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W,
                           X, logits, tok, ws, V, K, rb);
    else
        hipLaunchKernelGGL((head_q6k_kernel<2, 2>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W, X,
                           logits, tok, ws, V, K, rb);
    return check_launch("qkk_head_argmax");
}

int qkk_argmax(const float* logits, uint32_t* tok, uint32_t n, uint32_t batch, void* stream)
{
    if (!logits || !tok) return fail(QKK_EINVAL, "qkk_argmax: null pointer");
    if (n == 0 || batch == 0) return fail(QKK_EINVAL, "qkk_argmax: n and batch must be positive");
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(argmax_kernel, dim3(batch), dim3(256), 0, as_stream(stream), logits, tok, n);
    return check_launch("qkk_argmax");
}

} // extern "C"
