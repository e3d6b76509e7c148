// qk_gemv_lane.hip -- the quantised one-row GEMV with per-lane block loads.
//
// One wave covers 2048 consecutive weights of a row per pass (one lane = 32 weights) and every lane
// fetches its own block's fields from global memory with the widest load that covers them
// (LaneW<TYPE>::load), several rows before it starts the arithmetic.  This is the form of the kernel
// whose results and timings come from runs on an MI355X; qkk_gemv uses it unless the "one_row" switch
// selects the streaming form of qk_gemv.hip.
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {
namespace lane {

// ---- quantised GEMV ---------------------------------------------------------------------
// LPR   lanes per row (8..64): a row of K = 32*LPR*PASSES weights.
// PASSES how many 32*LPR slices a row has; x slices for all passes stay in registers.
// RIF   rows in flight per lane group: loads of RIF rows are issued before any arithmetic.
// DEEP  true: two register sets, the next chunk's loads in flight during the arithmetic of the
//       current one (large matrices); false: one chunk at a time (a wave has one or two chunks).
template <int TYPE, int LPR, int PASSES, int RIF, bool DEEP>
__global__ __launch_bounds__(256) void gemv_q_kernel(const uint8_t* __restrict__ W,
                                                     const float* __restrict__ X,
                                                     float* __restrict__ Y, uint32_t M, uint32_t K,
                                                     uint32_t row_bytes)
{
    __shared__ IqTables tab;
    constexpr bool TABLES = TYPE == QKK_IQ3_XXS || TYPE == QKK_IQ4_XS;
    // the codebook word travels with the first round trip (activations, first rows) and goes to LDS
    // after those loads are issued: a fill and a barrier up front would be a round trip of their own
    uint32_t grid_word = 0;
    if constexpr (TABLES) grid_word = g_iq3xxs_grid[threadIdx.x];
    constexpr int GROUPS = WAVE / LPR; // rows a wave works on side by side
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;

    XSlice xs[PASSES];
    float xsum[PASSES][4];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        load_xslice<TYPE>(xs[p], x + p * 32 * LPR, lir);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) s += xs[p].v[c * 8 + i];
            xsum[p][c] = s;
        }
    }
    const uint32_t pass_bytes = row_bytes / PASSES;

    // chunks of GROUPS*RIF rows are dealt round-robin to the waves of the (persistent) grid;
    // the loads of a wave's next chunk are issued before the arithmetic of the current one
    // (two register sets, loop unrolled by two, no branch around the loads: chunks past the
    // end re-read the last row and their results are dropped)
    constexpr uint32_t CHUNK = GROUPS * RIF;
    const uint32_t stride = gridDim.x * 4 * CHUNK;
    LaneW<TYPE> w[DEEP ? 2 : 1][RIF][PASSES];
    auto fetch = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            const uint32_t r = min(r0 + i * GROUPS + grp, M - 1);
#pragma unroll
            for (int p = 0; p < PASSES; p++)
                w[set][i][p].load(W + (size_t)r * row_bytes + (size_t)p * pass_bytes, lir);
        }
    };
    auto reduce = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) acc += w[set][i][p].dot(xs[p], xsum[p], &tab, lir);
            acc = lanes_sum<LPR>(acc);
            const uint32_t r = r0 + i * GROUPS + grp;
            if (lir == 0 && r < M) y[r] = acc;
        }
    };
    uint32_t r0 = (blockIdx.x * 4 + wave) * CHUNK;
    if constexpr (TABLES || DEEP) fetch(0, r0); // rows past the end re-read the last row
    if constexpr (TABLES) {
        tab.grid[threadIdx.x] = grid_word;
        if (threadIdx.x < 16) {
            constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) v = (int)threadIdx.x == i ? (float)kv[i] : v;
            tab.iq4[threadIdx.x] = v;
        }
        __syncthreads();
    }
    if constexpr (DEEP) {
        for (; r0 < M; r0 += 2 * stride) {
            fetch(1, r0 + stride);
            reduce(0, r0);
            fetch(0, r0 + 2 * stride);
            reduce(1, r0 + stride);
        }
    } else if constexpr (TABLES) { // the first chunk is already on its way
        while (r0 < M) {
            reduce(0, r0);
            r0 += stride;
            if (r0 < M) fetch(0, r0); // wave-uniform
        }
    } else {
        for (; r0 < M; r0 += stride) {
            fetch(0, r0);
            reduce(0, r0);
        }
    }
}


template <int TYPE, int LPR, int PASSES, int RIF>
static void launch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch,
                     uint32_t row_bytes, hipStream_t st)
{
    constexpr uint32_t CHUNK = WAVE / LPR * RIF;
    const uint32_t waves = (M + CHUNK - 1) / CHUNK;
    const dim3 grid(std::min((waves + 3) / 4, persistent_blocks()), batch);
    if (waves > 4 * grid.x * 4) // at least four chunks per wave: worth the second register set
        hipLaunchKernelGGL((gemv_q_kernel<TYPE, LPR, PASSES, RIF, true>), grid, dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, row_bytes);
    else
        hipLaunchKernelGGL((gemv_q_kernel<TYPE, LPR, PASSES, RIF, false>), grid, dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, row_bytes);
}

// true when the shape is one of the tiled ones and the launch was issued
template <int TYPE>
static bool dispatch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch, hipStream_t st)
{
    const uint32_t rb = (uint32_t)qkk_row_bytes(TYPE, K);
    // rows per wave: four where the matrix has rows enough to give every CU several waves that way,
    // fewer for short matrices (512 rows: 3.1-3.4 us with one row per wave against 4.6-5.2 us with four)
    // a layer's input projections as one matrix (12288 = qkv + gate, 9216 = q + k + v rows): M / 1024 rows
    // per wave make 256 workgroups, one per CU, where eight leave half the CUs with a second one
    if (K == 2048 && M == 12288 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 12>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M == 9216 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 9>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M >= 8192 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 8>(W, X, Y, M, K, batch, rb, st); // 7.5 -> 6.9 us
    else if (K == 2048 && M >= 2048) launch_q<TYPE, 64, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M >= 1024) launch_q<TYPE, 64, 1, 2>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048) launch_q<TYPE, 64, 1, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 4096 && M >= 1024) launch_q<TYPE, 64, 2, 2>(W, X, Y, M, K, batch, rb, st);
    else if (K == 4096) launch_q<TYPE, 64, 2, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 8192) launch_q<TYPE, 64, 4, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 1024) launch_q<TYPE, 32, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 512) launch_q<TYPE, 16, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 256) launch_q<TYPE, 8, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else return false;
    return true;
}

} // namespace lane

// The per-lane form of a quantised GEMV launch; false for a K outside the tiled shapes (the caller's
// one-wave-per-row kernel takes those).
bool lane_gemv_launch(int type, const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch, hipStream_t st)
{
    switch (type) {
    case QKK_Q8_0: return lane::dispatch_q<QKK_Q8_0>(W, X, Y, M, K, batch, st);
    case QKK_Q6_K: return lane::dispatch_q<QKK_Q6_K>(W, X, Y, M, K, batch, st);
    case QKK_IQ4_XS: return lane::dispatch_q<QKK_IQ4_XS>(W, X, Y, M, K, batch, st);
    case QKK_IQ3_XXS: return lane::dispatch_q<QKK_IQ3_XXS>(W, X, Y, M, K, batch, st);
    default: return false;
    }
}

} // namespace qk
