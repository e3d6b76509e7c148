// qk_head.hip -- LM head (Q6_K GEMV) with greedy sampling fused into the epilogue, and the
// stand-alone argmax.
//
// Each wave keeps the best (logit, id) of the rows it produced; a block folds its waves,
// writes one candidate, and the block that finishes last folds all candidates into the
// token id.  Ties go to the lower id; a logit must beat -3.4e38 to be chosen
// (reference shaders/argmax1.comp:25-33, argmax2.comp:20-28).
#include "qk_coop.h"
#include "qk_rows.h"
#include "qk_device.h"
#include "qk_host.h"
#include "qk_stream.h"

#include <stdlib.h>

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

// One activation row: the Q6_K rows are streamed as in the GEMV (qk_stream.h: chunks of RPC rows as
// 16-byte pieces through the wave's LDS area, the next chunk in flight during the arithmetic), and a
// wave keeps the best (logit, id) of its rows, which ascend, so a strict '>' keeps the lowest id.
// The vocabulary's rows behind the last full chunk are fetched per lane.
// NORM: the activation row is RMS-normalised with the weights nw on the way in (the output norm in
// front of the head): a wave holds all of x, so the mean square is one cross-lane sum; the dot products
// run on x * nw and the logits are scaled at the end.
template <int PASSES, int RPC, bool NORM = false>
__global__ __launch_bounds__(256) void head_q6k_kernel(const uint8_t* __restrict__ W,
                                                       const float* __restrict__ X,
                                                       float* __restrict__ logits_out,
                                                       uint32_t* __restrict__ tok, HeadWs ws, uint32_t V,
                                                       const float* __restrict__ nw, float eps)
{
    constexpr uint32_t K = 2048u * PASSES, RB = (uint32_t)qkk_row_bytes_dev<QKK_Q6_K>(K), PB = RB / PASSES;
    constexpr uint32_t CB = RPC * RB, NPC = CB / 16;
    constexpr int NP = (NPC + 63) / 64;
    static_assert(CB % 16 == 0, "a chunk of rows must be whole 16-byte pieces");
    __shared__ __attribute__((aligned(16))) uint8_t s_stage[4][WaveStage<NP>::AREA + 16];
    __shared__ float s_v[256];
    __shared__ uint32_t s_i[256];
    __shared__ uint32_t s_last;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t b = blockIdx.y;
    const float* x = X + (size_t)b * K;
    const uint32_t n_full = V / RPC, stride = gridDim.x * 4;
    uint32_t c = blockIdx.x * 4 + wave;

    WaveStage<NP> st;
    if (c < n_full) st.fetch(W + (size_t)c * CB, NPC, lane);
    XSlice xs[PASSES];
    float xsum[PASSES][4];
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        load_xslice<QKK_Q6_K>(xs[p], x + p * 2048, lane);
        if constexpr (NORM) {
            XSlice g;
            load_xslice<QKK_Q6_K>(g, nw + p * 2048, lane);
#pragma unroll
            for (int i = 0; i < 32; i++) {
                ss += xs[p].v[i] * xs[p].v[i];
                xs[p].v[i] *= g.v[i];
            }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            float t = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) t += xs[p].v[q * 8 + i];
            xsum[p][q] = t;
        }
    }
    float out_scale = 1.f;
    if constexpr (NORM) out_scale = 1.f / sqrtf(wave_sum(ss) / (float)K + eps);
    float bv = ARG_FLOOR;
    uint32_t bi = 0xFFFFFFFFu;
    auto take = [&](const LaneW<QKK_Q6_K> (&w)[PASSES], uint32_t r) {
        float acc = 0.f;
#pragma unroll
        for (int p = 0; p < PASSES; p++) acc += w[p].dot(xs[p], xsum[p], nullptr, lane);
        acc = wave_sum(acc) * out_scale;
        if (r < V) {
            if (logits_out && lane == 0) logits_out[(size_t)b * V + r] = acc;
            if (acc > bv) { bv = acc; bi = r; }
        }
    };
    uint8_t* area = s_stage[wave];
    vmem_drain(); // the activations are here: no wait for them inside the loop, behind the next chunk's loads
    for (; c < n_full; c += stride) {
        st.commit(area, lane);
        const uint32_t cn = c + stride;
        if (cn < n_full) st.fetch(W + (size_t)cn * CB, NPC, lane);
#pragma unroll
        for (int r = 0; r < RPC; r++) {
            LaneW<QKK_Q6_K> w[PASSES];
#pragma unroll
            for (int p = 0; p < PASSES; p++) lane_load_lds<QKK_Q6_K>(w[p], area, r * RB + p * PB, lane);
            take(w, c * RPC + r);
        }
    }
    // rows behind the last full chunk (they are the highest ids: still ascending for the wave that takes them last)
    for (uint32_t r = n_full * RPC + blockIdx.x * 4 + wave; r < V; r += stride) {
        LaneW<QKK_Q6_K> w[PASSES];
#pragma unroll
        for (int p = 0; p < PASSES; p++) w[p].load(W + (size_t)r * RB + (size_t)p * PB, lane);
        take(w, r);
    }

    // fold the four waves of the block
    if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 4; wv++)
            if (better(s_v[wv], s_i[wv], bv, bi)) { bv = s_v[wv]; bi = s_i[wv]; }
        publish(&ws.cand_v[(size_t)b * gridDim.x + blockIdx.x], bv);
        publish(&ws.cand_i[(size_t)b * gridDim.x + blockIdx.x], bi);
        s_last = arrive_last(&ws.counter[b], gridDim.x) ? 1u : 0u;
    }
    __syncthreads();
    if (s_last) {
        const uint32_t t = fold_candidates(ws.cand_v + (size_t)b * gridDim.x, ws.cand_i + (size_t)b * gridDim.x,
                                           gridDim.x, s_v, s_i);
        if (threadIdx.x == 0) {
            tok[b] = t;
            ws.counter[b] = 0u;
        }
    }
}

// The same head with per-lane block loads: every lane fetches its own block fields from global memory,
// RIF rows per wave in flight in two register sets.  The form whose results and timings come from runs
// on an MI355X (59-64 us for the 151,936-row head); used unless the "one_row" switch selects the
// streaming kernel above.
template <int PASSES, int RIF>
__global__ __launch_bounds__(256) void head_q6k_lane_kernel(const uint8_t* __restrict__ W,
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
    // chunks of RIF rows dealt round-robin to the waves; a wave's rows ascend.  The next
    // chunk's loads are issued before the arithmetic of the current one.
    const uint32_t stride = gridDim.x * 4 * RIF;
    LaneW<QKK_Q6_K> w[2][RIF][PASSES];
    auto fetch = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            const uint32_t r = min(r0 + i, V - 1);
#pragma unroll
            for (int p = 0; p < PASSES; p++)
                w[set][i][p].load(W + (size_t)r * row_bytes + (size_t)p * pass_bytes, lane);
        }
    };
    auto reduce = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) acc += w[set][i][p].dot(xs[p], xsum[p], nullptr, lane);
            acc = wave_sum(acc);
            const uint32_t r = r0 + i;
            if (r < V) {
                if (logits_out && lane == 0) logits_out[(size_t)b * V + r] = acc;
                if (acc > bv) { bv = acc; bi = r; } // rows ascend: strict '>' keeps the lowest id
            }
        }
    };
    uint32_t r0 = (blockIdx.x * 4 + wave) * RIF;
    fetch(0, r0);
    for (; r0 < V; r0 += 2 * stride) {
        fetch(1, r0 + stride);
        reduce(0, r0);
        fetch(0, r0 + 2 * stride);
        reduce(1, r0 + stride);
    }

    // fold the four waves of the block
    if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 4; wv++)
            if (better(s_v[wv], s_i[wv], bv, bi)) { bv = s_v[wv]; bi = s_i[wv]; }
        publish(&ws.cand_v[(size_t)b * gridDim.x + blockIdx.x], bv);
        publish(&ws.cand_i[(size_t)b * gridDim.x + blockIdx.x], bi);
        s_last = arrive_last(&ws.counter[b], gridDim.x) ? 1u : 0u;
    }
    __syncthreads();
    if (s_last) {
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

// ---- batched head: 2..16 rows of X against the Q6_K matrix on MFMA --------------------------
// The weights cross HBM once for the whole batch.  Workgroup = 16 waves sharing the batch's
// activations in LDS (hi/lo half planes in fragment order, 128 KiB for K = 2048); each wave
// streams 16-row tiles of W.  One Q6_K scale group (16 weights) is one 16x16x16 MFMA with the
// 6-bit integers as the weight operand; d*scale is applied to the MFMA result in fp32.
// Lane (row = l%16, g = l/16) fetches, per 256-weight block, the twelve dwords holding its
// 64 weights (4 per scale group), the 16 scales and d.
__device__ __forceinline__ void dpp_better(float& v, uint32_t& i)
{
#define QK_STEP(CTRL)                                                                             \
    {                                                                                             \
        const float ov = dpp_f<CTRL>(v);                                                          \
        const uint32_t oi = (uint32_t)dpp_i<CTRL>((int)i);                                        \
        if (better(ov, oi, v, i)) { v = ov; i = oi; }                                             \
    }
    QK_STEP(DPP_XOR1) QK_STEP(DPP_XOR2) QK_STEP(DPP_HALF_MIRROR) QK_STEP(DPP_MIRROR)
#undef QK_STEP
}

// ---- batch 2..16, K = 2048: the cooperative matrix-core stream (qk_coop.h) ------------------------
// The head is one dense "expert" of V rows applied to `batch` activation rows: every workgroup
// streams a contiguous range of row tiles, two per batch, and each thread keeps the best
// (logit, id) of the outputs it reduces (its rows ascend, so `>` keeps the lowest id).
constexpr int HEAD_TG = 2;
using HeadGeo = CoopGeom<QKK_Q6_K, 8, 1, HEAD_TG>;

__global__ __launch_bounds__(CT) void head_q6k_coop_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                           float* __restrict__ logits_out, uint32_t* __restrict__ tok,
                                                           HeadWs ws, uint32_t V, uint32_t batch)
{
    constexpr uint32_t K = 2048, ROW = HeadGeo::RB, BT = HeadGeo::BT;
    static_assert(BT * 256 <= CT, "one output per thread and batch");
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    fill_mfma_tables(tab, tid, CT);

    // batches [b0, b1) of the tensor's `total`, an even split (b1 <= total for every workgroup)
    const uint32_t total = (V + 16 * BT - 1) / (16 * BT);
    const uint32_t b0 = (uint32_t)((uint64_t)blockIdx.x * total / gridDim.x);
    const uint32_t b1 = (uint32_t)((uint64_t)(blockIdx.x + 1) * total / gridDim.x);
    const uint32_t row0 = b0 * BT * 16;
    const uint32_t nb = row0 < V ? b1 - b0 : 0u;
    float bv = ARG_FLOOR;
    uint32_t bi = 0xFFFFFFFFu;
    __syncthreads();
    if (nb) {
        coop_stream<QKK_Q6_K, 8, 1, HEAD_TG, false, true>(
            W + (size_t)row0 * ROW, nullptr, nb, X, K, batch, [](uint32_t r) { return r; }, smem, tab, tid,
            [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float, uint32_t) {
                const uint32_t t = 4 * (ln >> 4) + e, row = row0 + tile * 16 + (ln & 15u);
                if (t < batch && row < V) {
                    if (logits_out) logits_out[(size_t)t * V + row] = sum0;
                    if (sum0 > bv) { bv = sum0; bi = row; }
                }
            },
            (size_t)V * ROW - 16 - (size_t)row0 * ROW);
    }
    // per token: the 32 threads that reduce its outputs (16 rows x BT tiles), then the workgroups
    float* s_v = (float*)smem;
    uint32_t* s_i = (uint32_t*)(smem + CT * 4);
    s_v[tid] = bv;
    s_i[tid] = bi;
    __syncthreads();
    if ((uint32_t)tid < batch) {
        float v = ARG_FLOOR;
        uint32_t i = 0xFFFFFFFFu;
        const uint32_t g = tid >> 2, e = tid & 3u;
        for (uint32_t bt = 0; bt < BT; bt++)
            for (uint32_t j = 0; j < 16; j++) {
                const uint32_t o = bt * 256 + e * 64 + g * 16 + j;
                if (better(s_v[o], s_i[o], v, i)) { v = s_v[o]; i = s_i[o]; }
            }
        publish(&ws.cand_v[(size_t)tid * gridDim.x + blockIdx.x], v);
        publish(&ws.cand_i[(size_t)tid * gridDim.x + blockIdx.x], i);
        publish_wait(); // acknowledged before the barrier and the arrival count
    }
    __syncthreads();
    if (tid == 0) s_last = arrive_last(&ws.counter[0], gridDim.x) ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        // one wave per token folds the workgroups' candidates
        for (uint32_t t = wave; t < batch; t += CW) {
            float v = ARG_FLOOR;
            uint32_t i = 0xFFFFFFFFu;
            for (uint32_t c = lane; c < gridDim.x; c += 64) {
                const float cv = ws.cand_v[(size_t)t * gridDim.x + c];
                const uint32_t ci = ws.cand_i[(size_t)t * gridDim.x + c];
                if (better(cv, ci, v, i)) { v = cv; i = ci; }
            }
            dpp_better(v, i);
            // four rows of 16 lanes remain
            float fv = readlane_f(v, 0);
            uint32_t fi = (uint32_t)__builtin_amdgcn_readlane((int)i, 0);
#pragma unroll
            for (int r = 16; r < 64; r += 16) {
                const float ov = readlane_f(v, r);
                const uint32_t oi = (uint32_t)__builtin_amdgcn_readlane((int)i, r);
                if (better(ov, oi, fv, fi)) { fv = ov; fi = oi; }
            }
            if (lane == 0) tok[t] = fi == 0xFFFFFFFFu ? 0u : fi;
        }
        if (tid == 0) ws.counter[0] = 0u;
    }
}

// ---- 2..16 rows with the waves splitting the vocabulary rows (the "head_rows" switch) ----
// The cooperative stream above splits K over the waves: per batch of 32 vocabulary rows partial tiles go through
// LDS, one wave sums them and a barrier closes the batch -- 4,748 batches for the 151,936-row head, and it is
// that fixed cost per batch which holds 16 rows at a third of the memory roofline.  Here a work item is a block
// of 128 vocabulary rows and a wave owns 16 of them for all of K (rows_stream, qk_rows.h): its accumulators are
// logits, a thread keeps the best (logit, id) of each of its four activation rows across its items (its rows
// ascend, so `>` keeps the lowest id), and the fold over the workgroup, the candidates and the last workgroup are
// those of the kernel above.  64 KB of LDS, two workgroups per CU.
__global__ __launch_bounds__(MR_THREADS, 4) void head_q6k_rows_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                                      float* __restrict__ logits_out, uint32_t* __restrict__ tok,
                                                                      HeadWs ws, uint32_t V, uint32_t batch)
{
    using G = RowsGeo<QKK_Q6_K, 1>;
    constexpr uint32_t K = 2048, ROW = (K / 256) * G::FB;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab; // Q6_K reads no table; rows_stream takes the reference
    __shared__ uint32_t s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, g = lane >> 4;
    const size_t last_piece = (size_t)V * ROW - 16; // a Q6_K row of 2048 is 105 pieces: the tensor ends on one
    const uint32_t items = (V + MR_ROWS - 1) / MR_ROWS;
    const float* arow = X + (size_t)min((uint32_t)j, batch - 1) * K; // operand rows behind the batch repeat its last row
    float bv[4];
    uint32_t bi[4];
#pragma unroll
    for (int e = 0; e < 4; e++) { bv[e] = ARG_FLOOR; bi[e] = 0xFFFFFFFFu; }
    // this workgroup's items blockIdx.x, blockIdx.x + gridDim.x, ... as one pipeline
    const uint32_t mine = blockIdx.x < items ? (items - blockIdx.x + gridDim.x - 1) / gridDim.x : 0u;
    if (mine)
        rows_stream<QKK_Q6_K, 1>(
            W, nullptr, mine, [&](uint32_t b) { return (size_t)(blockIdx.x + b * gridDim.x) * MR_ROWS * ROW; }, ROW, last_piece, K / 256,
            arow, smem, tab, tid, [&](uint32_t b, const float4v(&acc)[1]) {
                const uint32_t row = (blockIdx.x + b * gridDim.x) * MR_ROWS + 16 * wave + j; // rows behind V were read from clamped addresses: dropped here
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t t = 4 * g + e;
                    if (t < batch && row < V) {
                        if (logits_out) logits_out[(size_t)t * V + row] = acc[0][e];
                        if (acc[0][e] > bv[e]) { bv[e] = acc[0][e]; bi[e] = row; }
                    }
                }
            });
    __syncthreads();
    // per activation row: the 128 threads that hold its outputs (16 rows x 8 waves), then the workgroups
    float* s_v = (float*)smem;
    uint32_t* s_i = (uint32_t*)(smem + MR_THREADS * 4 * 4);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        s_v[tid * 4 + e] = bv[e];
        s_i[tid * 4 + e] = bi[e];
    }
    __syncthreads();
    if ((uint32_t)tid < batch) {
        float v = ARG_FLOOR;
        uint32_t i = 0xFFFFFFFFu;
        const uint32_t tg = tid >> 2, te = tid & 3u;
        for (uint32_t w = 0; w < MR_THREADS / 64; w++)
            for (uint32_t jj = 0; jj < 16; jj++) {
                const uint32_t o = (w * 64 + tg * 16 + jj) * 4 + te;
                if (better(s_v[o], s_i[o], v, i)) { v = s_v[o]; i = s_i[o]; }
            }
        publish(&ws.cand_v[(size_t)tid * gridDim.x + blockIdx.x], v);
        publish(&ws.cand_i[(size_t)tid * gridDim.x + blockIdx.x], i);
        publish_wait(); // acknowledged before the barrier and the arrival count
    }
    __syncthreads();
    if (tid == 0) s_last = arrive_last(&ws.counter[0], gridDim.x) ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        // one wave per activation row folds the workgroups' candidates
        for (uint32_t t = wave; t < batch; t += MR_THREADS / 64) {
            float v = ARG_FLOOR;
            uint32_t i = 0xFFFFFFFFu;
            for (uint32_t c = lane; c < gridDim.x; c += 64) {
                const float cv = ws.cand_v[(size_t)t * gridDim.x + c];
                const uint32_t ci = ws.cand_i[(size_t)t * gridDim.x + c];
                if (better(cv, ci, v, i)) { v = cv; i = ci; }
            }
            dpp_better(v, i);
            // four rows of 16 lanes remain
            float fv = readlane_f(v, 0);
            uint32_t fi = (uint32_t)__builtin_amdgcn_readlane((int)i, 0);
#pragma unroll
            for (int r = 16; r < 64; r += 16) {
                const float ov = readlane_f(v, r);
                const uint32_t oi = (uint32_t)__builtin_amdgcn_readlane((int)i, r);
                if (better(ov, oi, fv, fi)) { fv = ov; fi = oi; }
            }
            if (lane == 0) tok[t] = fi == 0xFFFFFFFFu ? 0u : fi;
        }
        if (tid == 0) ws.counter[0] = 0u;
    }
}

// Grid of the one-row kernel: one chunk per wave for a small vocabulary, else a persistent grid eight
// workgroups deep per CU (16 KB of LDS each), the depth at which the same streaming loop read Q6_K
// fastest as a plain GEMV.
constexpr uint32_t HEAD_RPC = 2, HEAD_DEPTH = 8;
static uint32_t head_blocks(uint32_t V, uint32_t rpc)
{
    // the "head_depth" switch (1..8): workgroups per CU, for sweeps on the device (never more than the workspace bound's 8)
    const uint32_t depth_env = (uint32_t)options().head_depth;
    const uint32_t waves = std::max(V / rpc, V % rpc);
    return std::max(1u, std::min((waves + 3) / 4, persistent_blocks() / 4 * (depth_env ? depth_env : HEAD_DEPTH)));
}

// Persistent grid of the per-lane kernel.  Measured on the 151,936-row head (two rows in flight per
// wave, double-buffered): 256 workgroups 65.0 us, 512: 60.0, 768: 62.4, 1024: 63.2, and grids that
// are not a multiple of the CU count lose 5 us more; four rows in flight (133 VGPRs) 68.3 us.
constexpr uint32_t HEAD_LANE_RIF = 2;
static uint32_t head_lane_blocks(uint32_t V, uint32_t rif)
{
    const uint32_t waves = (V + rif - 1) / rif;
    return std::min((waves + 3) / 4, persistent_blocks() / 2);
}

} // namespace qk

using namespace qk;

extern "C" {

size_t qkk_head_workspace_bytes(uint32_t V, uint32_t batch)
{
    if (V == 0 || batch == 0) return 0;
    const size_t blocks = std::max<size_t>(head_blocks(V, 1), persistent_blocks() / 2); // upper bound over the kernels
    return 256 + (size_t)batch * blocks * 8;
}

static int head_argmax_impl(const void* W, const float* X, uint32_t* tok, float* logits, uint32_t V, uint32_t K,
                            uint32_t batch, void* workspace, size_t workspace_bytes, void* stream,
                            const float* w_norm, float eps)
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
    if (w_norm && (batch != 1 || K != 2048))
        return fail(QKK_ESHAPE, "qkk_head_argmax_norm: one row of 2048 (got %u rows of %u)", batch, K);
    if (batch >= 2 && batch <= 16 && K == 2048 && options().head_rows) {
        // the "head_rows" switch: blocks of 128 vocabulary rows, a wave owning 16 of them for all of K
        using RG = RowsGeo<QKK_Q6_K, 1>;
        HeadWs ws;
        const uint32_t blocks = std::min((V + MR_ROWS - 1) / MR_ROWS, persistent_blocks() / 2); // two workgroups per CU (LDS)
        ws.counter = (uint32_t*)workspace;
        ws.cand_v = (float*)((uint8_t*)workspace + 256);
        ws.cand_i = (uint32_t*)(ws.cand_v + (size_t)batch * blocks);
        static const bool raised = ((void)hipFuncSetAttribute((const void*)head_q6k_rows_kernel,
                                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)RG::LDS_BYTES), true);
        (void)raised;
        hipLaunchKernelGGL(head_q6k_rows_kernel, dim3(blocks), dim3(MR_THREADS), RG::LDS_BYTES, st, (const uint8_t*)W, X, logits,
                           tok, ws, V, batch);
        return check_launch("qkk_head_argmax");
    }
    if (batch >= 2 && batch <= 16 && K == 2048) {
        HeadWs ws;
        const uint32_t blocks = persistent_blocks() / 4; // one workgroup per CU (LDS)
        ws.counter = (uint32_t*)workspace;
        ws.cand_v = (float*)((uint8_t*)workspace + 256);
        ws.cand_i = (uint32_t*)(ws.cand_v + (size_t)batch * blocks);
        static bool attr_done = false;
        if (!attr_done) {
            (void)hipFuncSetAttribute((const void*)head_q6k_coop_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)HeadGeo::LDS_BYTES);
            attr_done = true;
        }
        hipLaunchKernelGGL(head_q6k_coop_kernel, dim3(blocks), dim3(CT), HeadGeo::LDS_BYTES, st, (const uint8_t*)W, X,
                           logits, tok, ws, V, batch);
        return check_launch("qkk_head_argmax");
    }
    const bool lane_form = !w_norm && !options().one_row_stream; // the norm in front exists in the streaming form only
    const uint32_t blocks = lane_form ? head_lane_blocks(V, HEAD_LANE_RIF) : head_blocks(V, K == 2048 ? HEAD_RPC : 1);
    HeadWs ws;
    ws.counter = (uint32_t*)workspace;
    ws.cand_v = (float*)((uint8_t*)workspace + 256);
    ws.cand_i = (uint32_t*)(ws.cand_v + (size_t)batch * blocks);
    if (lane_form) {
        const uint32_t rb = (uint32_t)qkk_row_bytes(QKK_Q6_K, K);
        if (K == 2048)
            hipLaunchKernelGGL((head_q6k_lane_kernel<1, HEAD_LANE_RIF>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W,
                               X, logits, tok, ws, V, K, rb);
        else
            hipLaunchKernelGGL((head_q6k_lane_kernel<2, 2>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W, X,
                               logits, tok, ws, V, K, rb);
    } else if (w_norm)
        hipLaunchKernelGGL((head_q6k_kernel<1, HEAD_RPC, true>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W,
                           X, logits, tok, ws, V, w_norm, eps);
    else if (K == 2048)
        hipLaunchKernelGGL((head_q6k_kernel<1, HEAD_RPC>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W,
                           X, logits, tok, ws, V, (const float*)nullptr, 0.f);
    else
        hipLaunchKernelGGL((head_q6k_kernel<2, 1>), dim3(blocks, batch), dim3(256), 0, st, (const uint8_t*)W, X,
                           logits, tok, ws, V, (const float*)nullptr, 0.f);
    return check_launch("qkk_head_argmax");
}

int qkk_head_argmax(const void* W, const float* X, uint32_t* tok, float* logits, uint32_t V, uint32_t K,
                    uint32_t batch, void* workspace, size_t workspace_bytes, void* stream)
{
    return head_argmax_impl(W, X, tok, logits, V, K, batch, workspace, workspace_bytes, stream, nullptr, 0.f);
}

int qkk_head_argmax_norm(const void* W, const float* X, const float* w_norm, float eps, uint32_t* tok, float* logits,
                         uint32_t V, uint32_t K, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!w_norm || !aligned16(w_norm)) return fail(QKK_EINVAL, "qkk_head_argmax_norm: w_norm must be a 16-byte aligned pointer");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_head_argmax_norm: eps must be non-negative");
    return head_argmax_impl(W, X, tok, logits, V, K, 1, workspace, workspace_bytes, stream, w_norm, eps);
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
