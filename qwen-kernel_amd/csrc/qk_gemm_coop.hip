// qk_gemm_coop.hip -- Y[n][m] = W[m] . X[n] for several activation rows on the cooperative
// matrix-core stream (qk_coop.h): the weights (any of the four block formats) are read once
// for all rows instead of once per row.  Serves qkk_gemm_q8_0 (batched prefill; reference
// shaders/gemm_q8_0.comp:32-101) and qkk_gemv with batch >= 2 (the z-batched decode GEMVs of
// reference src/main.cpp:4310-4335, which re-read the weights per slot).
#include "qk_coop.h"
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {

// The projection is one dense "expert" of M rows.  A workgroup takes a range of row tiles and
// NA*16 activation rows; every weight fragment is decoded once and applied to all NA activation
// tiles the wave keeps in registers.  K = 256*KS*KP: with KP > 1 the workgroup streams its rows
// KP times, one K range of 256*KS weights per pass (strided rows), reloads its activation slice
// for the range, and the same thread adds each pass's sum to what it stored the pass before --
// a fixed order, so results stay bit-reproducible, and every weight byte is still read once.
template <int TYPE, int KS, int NA>
using GemmGeo = CoopGeom<TYPE, KS, 1, 1, false, NA>;

template <int TYPE, int KS, int NA, int KP>
__global__ __launch_bounds__(CT) void gemm_coop_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                       float* __restrict__ Y, uint32_t M, uint32_t N, uint32_t ranges)
{
    using Geo = GemmGeo<TYPE, KS, NA>;
    constexpr uint32_t KPART = 256 * KS, K = KPART * KP, RB = Geo::RB, RBF = RB * KP, BT = Geo::BT;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    const int tid = threadIdx.x;
    fill_mfma_tables_for<TYPE>(tab, tid, CT); // in place before the stream's first barrier
    const uint32_t groups = (N + 16 * NA - 1) / (16 * NA);
    const uint32_t q = blockIdx.x % groups, r = blockIdx.x / groups;
    // batches [b0, b1) of the tensor's `total`, an even split over the ranges (b1 <= total)
    const uint32_t total = (M + 16 * BT - 1) / (16 * BT);
    const uint32_t b0 = (uint32_t)((uint64_t)r * total / ranges), b1 = (uint32_t)((uint64_t)(r + 1) * total / ranges);
    const uint32_t row0 = b0 * BT * 16, tok0 = q * 16 * NA;
    if (b1 <= b0 || row0 >= M || tok0 >= N) return; // the whole workgroup
    const uint32_t np = min((uint32_t)(16 * NA), N - tok0);
    if constexpr (KP == 1) {
        coop_stream<TYPE, KS, 1, 1, false, true, NA>(
            W + (size_t)row0 * RB, nullptr, b1 - b0, X + (size_t)tok0 * K, K, np, [](uint32_t t) { return t; }, smem, tab, tid,
            [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float, uint32_t na) {
                const uint32_t t = 16 * na + 4 * (ln >> 4) + e, row = row0 + tile * 16 + (ln & 15u);
                if (t < np && row < M) Y[(size_t)(tok0 + t) * M + row] = sum0;
            },
            (size_t)M * RB - 16 - (size_t)row0 * RB);
    } else {
#pragma unroll 1
        for (uint32_t kp = 0; kp < (uint32_t)KP; kp++) {
            const size_t base = (size_t)row0 * RBF + (size_t)kp * RB; // first row of the range, K range kp
            coop_stream<TYPE, KS, 1, 1, false, true, NA, 2, true>(
                W + base, nullptr, b1 - b0, X + (size_t)tok0 * K + kp * KPART, K, np, [](uint32_t t) { return t; }, smem,
                tab, tid,
                [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float, uint32_t na) {
                    const uint32_t t = 16 * na + 4 * (ln >> 4) + e, row = row0 + tile * 16 + (ln & 15u);
                    if (t < np && row < M) {
                        float* y = Y + (size_t)(tok0 + t) * M + row;
                        *y = kp ? *y + sum0 : sum0;
                    }
                },
                (size_t)M * RBF - 16 - base, RBF);
        }
    }
}

template <int TYPE, int KS, int NA, int KP>
static void launch(const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t N, hipStream_t st)
{
    using Geo = GemmGeo<TYPE, KS, NA>;
    // workgroups that fit a CU at once (registers, LDS): one or two
    static const uint32_t per_cu = [] {
        (void)hipFuncSetAttribute((const void*)gemm_coop_kernel<TYPE, KS, NA, KP>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)Geo::LDS_BYTES);
        int n = 1;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)gemm_coop_kernel<TYPE, KS, NA, KP>, CT,
                                                         Geo::LDS_BYTES) != hipSuccess || n < 1)
            n = 1;
        return (uint32_t)std::min(n, 2);
    }();
    const uint32_t groups = (N + 16 * NA - 1) / (16 * NA);
    const uint32_t total = (M + 16 * Geo::BT - 1) / (16 * Geo::BT);
    // fill the CUs once; a tensor with no more batches than CUs gets a workgroup per batch (the fixed
    // cost of a workgroup dominates there), a larger one at least two batches per workgroup
    const uint32_t want = std::max(1u, per_cu * (persistent_blocks() / 4) / groups);
    const uint32_t minb = total <= persistent_blocks() / 4 ? 1u : 2u;
    const uint32_t ranges = std::max(1u, std::min(want, (total + minb - 1) / minb));
    hipLaunchKernelGGL((gemm_coop_kernel<TYPE, KS, NA, KP>), dim3(groups * ranges), dim3(CT), Geo::LDS_BYTES, st, W, X, Y,
                       M, N, ranges);
}

template <int TYPE, int KS, int KP = 1>
static void launch_na(const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t N, hipStream_t st)
{
    if (N <= 16) launch<TYPE, KS, 1, KP>(W, X, Y, M, N, st);
    else launch<TYPE, KS, 2, KP>(W, X, Y, M, N, st);
}

template <int TYPE>
static bool launch_k(const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N, hipStream_t st)
{
    switch (K) {
    case 256: launch_na<TYPE, 1>(W, X, Y, M, N, st); return true;
    case 512: launch_na<TYPE, 2>(W, X, Y, M, N, st); return true;
    case 1024: launch_na<TYPE, 4>(W, X, Y, M, N, st); return true;
    case 2048: launch_na<TYPE, 8>(W, X, Y, M, N, st); return true;
    case 4096: launch_na<TYPE, 8, 2>(W, X, Y, M, N, st); return true;
    default: return false;
    }
}

bool tiled_gemm_launch(int type, const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N, hipStream_t st); // qk_gemm_tiled.hip

bool coop_gemm_launch(int type, const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N,
                      hipStream_t st)
{
    // the "gemm_tiled" switch: 64 rows and more through the kernel that decodes every weight tile once per 128 rows
    if (options().gemm_tiled && tiled_gemm_launch(type, W, X, Y, M, K, N, st)) return true;
    // the stream copies whole 16-byte pieces: the tensor must end on one
    if (((uint64_t)M * qkk_row_bytes(type, K)) % 16) return false;
    switch (type) {
    case QKK_Q8_0: return launch_k<QKK_Q8_0>(W, X, Y, M, K, N, st);
    case QKK_Q6_K: return launch_k<QKK_Q6_K>(W, X, Y, M, K, N, st);
    case QKK_IQ4_XS: return launch_k<QKK_IQ4_XS>(W, X, Y, M, K, N, st);
    case QKK_IQ3_XXS: return launch_k<QKK_IQ3_XXS>(W, X, Y, M, K, N, st);
    default: return false;
    }
}

} // namespace qk
