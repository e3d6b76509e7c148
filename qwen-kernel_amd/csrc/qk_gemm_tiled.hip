// qk_gemm_tiled.hip -- Y[n][m] = W[m] . X[n] for a prompt's worth of activation rows (64 and more):
// every weight tile is fetched and decoded ONCE for 128 rows.
//
// The cooperative stream of qk_gemm_coop.hip is activation-stationary: a wave keeps its K slice of at
// most 32 activation rows in registers and the workgroup's waves split K, so 128 rows stream and decode
// every weight tile four times and pay a cross-wave sum per 16 weight rows.  This kernel turns the
// product round (the counterpart of the 128 x 64 tile of reference shaders/gemm_q8_0_coopmat2.comp:42-148):
// a workgroup owns 32 weight rows and 128 activation rows for ALL of K; its eight waves take 16
// activation rows each and both 16-row weight tiles, so nothing is summed across waves and a lane's
// accumulators are its outputs.  Per K step of 256 weights the workgroup copies the 32 rows' blocks to LDS
// (aligned 16-byte pieces that cover each row's fragment wherever it starts, the next step's pieces in
// flight during the arithmetic, two buffers, one barrier per step), every wave decodes them with
// BFrag<TYPE>::step -- the decoder of the cooperative stream, so all four block formats and the same
// exactness: activations hi + lo, weights hi (+ lo where the product with the sub-scale does not fit a
// half), three (two) v_mfma_f32_16x16x32_f16 per product -- against its own activation operand, which it
// loads and splits for the next step while the matrix cores run this one.
// Behind the "gemm_tiled" switch until it has been run and timed on a device.
#include "qk_coop.h"
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {

constexpr uint32_t GT_BM = 32, GT_BN = 128, GT_THREADS = 512; // weight rows, activation rows, threads of a workgroup

// The activation operand of one wave for one K step as loaded (fp32, in the cut of `LAYOUT`, see BFrag):
// kept apart from its conversion so that the loads of the next step are in flight during this step's MFMAs.
struct ARaw {
    float4 v[8][2];
};
template <int LAYOUT>
__device__ __forceinline__ void load_araw(ARaw& r, const float* __restrict__ row, uint32_t k0, int g)
{
#pragma unroll
    for (int i = 0; i < 8; i++) {
        // LAYOUT 2: K in its natural order, step i = weights 32 i .. 32 i + 31 (one Q8_0 block), group g eight of them
        const uint32_t k = LAYOUT == 2 ? 32 * i + 8 * g
                         : LAYOUT == 0 ? 64 * g + 8 * i : 128 * (g >> 1) + 32 * (i >> 1) + 16 * (g & 1) + 8 * (i & 1);
        r.v[i][0] = *(const float4*)(row + k0 + k);
        r.v[i][1] = *(const float4*)(row + k0 + k + 4);
    }
}
// x = hi + lo.  Rows behind the last activation row repeat it (the loads are clamped): an output depends on
// its own activation row only and those outputs are not stored, so nothing needs to be zeroed.
// `one` is 1.0 in a register the compiler cannot see through: x * one - hi is then a genuine fused
// multiply-add with mixed operands, which has a one-instruction form with a half result (v_fma_mixlo_f16);
// written as x - hi it becomes a conversion, a subtraction and another conversion.
__device__ __forceinline__ void split_araw(AFrag& a, const ARaw& r, float one)
{
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float f[8] = {r.v[i][0].x, r.v[i][0].y, r.v[i][0].z, r.v[i][0].w, r.v[i][1].x, r.v[i][1].y, r.v[i][1].z, r.v[i][1].w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            a.hi[i][e] = (_Float16)f[e];
            a.lo[i][e] = (_Float16)__builtin_fmaf(f[e], one, -(float)a.hi[i][e]);
        }
    }
}

// Q8_0 has a cut of its own: one matrix instruction's K = 32 is exactly one block, so the operand holds the
// block's integers as they are (exact in a half, no residual operand), two instructions (activations hi, lo)
// fill a fresh 16 x 16 result, and the block's scale multiplies that result in fp32 -- two matrix instructions
// per product instead of three and a decode of 6 vector operations per block and tile instead of 18.
struct Q8Rows {
    uint2 q[8];     // this lane's eight weights of each of the fragment's eight blocks
    uint32_t d[8];  // the blocks' scales (half bits)
    __device__ __forceinline__ void load(const uint8_t* frag, int g)
    {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            d[i] = ldg<uint16_t>(frag + i * Q8_0_BYTES);
            q[i] = ldg<uint2>(frag + i * Q8_0_BYTES + 2 + 8 * g);
        }
    }
    __device__ __forceinline__ half8 block(int i) const
    {
        const half4 a = bytes_to_half4(q[i].x ^ 0x80808080u, 128.f), b = bytes_to_half4(q[i].y ^ 0x80808080u, 128.f);
        return half8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    }
    __device__ __forceinline__ float scale(int i) const { return h2f((uint16_t)d[i]); }
};

template <int TYPE>
__global__ __launch_bounds__(GT_THREADS) void gemm_tiled_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                               float* __restrict__ Y, uint32_t M, uint32_t N, uint32_t K)
{
    using F = BFrag<TYPE>;
    constexpr uint32_t FB = F::BYTES;                 // bytes of a row's 256-weight fragment
    constexpr uint32_t NPW = (FB + 15 + 15) / 16;     // 16-byte pieces that cover a fragment wherever it starts
    constexpr uint32_t WIN = NPW * 16, PIECES = GT_BM * NPW;
    constexpr int NLD = (PIECES + GT_THREADS - 1) / GT_THREADS;
    __shared__ __attribute__((aligned(16))) uint8_t s_raw[2][GT_BM * WIN + 16];
    __shared__ MfmaTables tab;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, g = lane >> 4;
    fill_mfma_tables_for<TYPE>(tab, tid, GT_THREADS); // in place before the first barrier
    const uint32_t nfrag = K / 256;
    const size_t stride = (size_t)nfrag * FB;         // bytes of a weight row
    const size_t last_piece = (size_t)M * stride - 16; // the tensor ends on a 16-byte boundary (the launcher checks)
    const uint32_t row0 = blockIdx.x * GT_BM;
    const uint32_t tok = blockIdx.y * GT_BN + wave * 16 + j; // this lane's activation row of the A operand
    const bool wave_live = blockIdx.y * GT_BN + wave * 16 < N; // wave-uniform: its 16 rows exist at least in part
    const float* xrow = X + (size_t)min(tok, N - 1) * K;
    float one = 1.f; // in a register the compiler cannot see through (see split_araw)
    asm volatile("" : QK_REG(one));

    // piece p of a K step: row p / NPW of the block, piece p % NPW of that row's window; rows behind the
    // matrix repeat its last row, pieces behind the tensor its last piece (neither is used)
    size_t src[NLD];          // where the piece's row starts in the tensor
    uint32_t pq[NLD], dst[NLD]; // its number inside the row's window, its place in LDS
#pragma unroll
    for (int n = 0; n < NLD; n++) {
        const uint32_t p = min((uint32_t)(tid + GT_THREADS * n), PIECES - 1);
        const uint32_t r = p / NPW;
        pq[n] = p % NPW;
        src[n] = (size_t)min(row0 + r, M - 1) * stride;
        dst[n] = r * WIN + pq[n] * 16;
    }
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 ld[NLD];
    const auto fetch = [&](uint32_t f) {
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            const size_t at = src[n] + (size_t)f * FB; // the row's fragment f; its window starts at the 16-byte boundary below
            ld[n] = *(const u32x4*)(W + min((at & ~(size_t)15) + 16u * pq[n], last_piece));
        }
    };
    const auto commit = [&](uint32_t buf) {
#pragma unroll
        for (int n = 0; n < NLD; n++)
            if (PIECES % GT_THREADS == 0 || n + 1 < NLD || tid + GT_THREADS * n < PIECES) *(u32x4*)(s_raw[buf] + dst[n]) = ld[n];
    };
    // where this lane's weight rows (row 16 t + j of the block, t = 0, 1) start inside their windows
    const auto frag_at = [&](uint32_t buf, uint32_t t, uint32_t f) -> const uint8_t* {
        const size_t at = (size_t)min(row0 + 16 * t + j, M - 1) * stride + (size_t)f * FB;
        return s_raw[buf] + (16 * t + j) * WIN + (at & 15);
    };

    fetch(0);
    ARaw raw;
    AFrag a;
    constexpr int CUT = TYPE == QKK_Q8_0 ? 2 : F::LAYOUT; // how K is dealt to the steps and lane groups
    if (wave_live) load_araw<CUT>(raw, xrow, 0, g);
    commit(0);
    if (wave_live) split_araw(a, raw, one);
    __syncthreads();

    float4v acc[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll 1
    for (uint32_t f = 0; f < nfrag; f++) {
        const uint32_t buf = f & 1u, fn = min(f + 1, nfrag - 1); // past the end: a harmless re-read
        fetch(fn);
        if (wave_live) load_araw<CUT>(raw, xrow, 256 * fn, g);
        if constexpr (TYPE == QKK_Q8_0) {
            if (wave_live) {
                Q8Rows w[2];
#pragma unroll
                for (int t = 0; t < 2; t++) w[t].load(frag_at(buf, t, f), g);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4v zero = {0.f, 0.f, 0.f, 0.f};
                    half8 b[2];
                    float4v blk[2];
#pragma unroll
                    for (int t = 0; t < 2; t++) b[t] = w[t].block(i);
#pragma unroll
                    for (int t = 0; t < 2; t++) blk[t] = mfma16x32(a.hi[i], b[t], zero);
#pragma unroll
                    for (int t = 0; t < 2; t++) blk[t] = mfma16x32(a.lo[i], b[t], blk[t]);
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const float sc = w[t].scale(i);
                        acc[t] += float4v{sc * blk[t][0], sc * blk[t][1], sc * blk[t][2], sc * blk[t][3]};
                    }
                }
                split_araw(a, raw, one);
            }
        } else if (wave_live) {
            F w[2];
#pragma unroll
            for (int t = 0; t < 2; t++) w[t].load(frag_at(buf, t, f), 0, g);
            float4v part[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                half8 bl[2], bh[2];
#pragma unroll
                for (int t = 0; t < 2; t++) bh[t] = w[t].step(i, g, tab, bl[t]);
                // the two tiles' chains take turns, so that a matrix instruction does not wait for the one before it
#pragma unroll
                for (int t = 0; t < 2; t++) part[t] = mfma16x32(a.hi[i], bh[t], part[t]);
#pragma unroll
                for (int t = 0; t < 2; t++) part[t] = mfma16x32(a.lo[i], bh[t], part[t]);
                if constexpr (F::SPLIT) {
#pragma unroll
                    for (int t = 0; t < 2; t++) part[t] = mfma16x32(a.hi[i], bl[t], part[t]);
                }
                __builtin_amdgcn_sched_barrier(0); // keep the decode of later steps from piling up in registers
            }
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const float sc = w[t].post(); // the row's fp16 scale of this fragment, in fp32
                acc[t] += float4v{sc * part[t][0], sc * part[t][1], sc * part[t][2], sc * part[t][3]};
            }
            split_araw(a, raw, one); // the next step's operand
        }
        commit(buf ^ 1u);
        __syncthreads(); // step f is read, step f + 1 is in place
    }
    if (!wave_live) return;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint32_t row = row0 + 16 * t + j;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t n = blockIdx.y * GT_BN + wave * 16 + 4 * g + e; // D[4 g + e][j]
            if (row < M && n < N) Y[(size_t)n * M + row] = acc[t][e];
        }
    }
}

// true when the shape is one this kernel covers and the launch was issued
bool tiled_gemm_launch(int type, const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N, hipStream_t st)
{
    if (N < 64 || K % 256 || K == 0 || ((uint64_t)M * qkk_row_bytes(type, K)) % 16) return false;
    const dim3 grid((M + GT_BM - 1) / GT_BM, (N + GT_BN - 1) / GT_BN);
    if (grid.y > 65535) return false;
    switch (type) {
    case QKK_Q8_0: hipLaunchKernelGGL(gemm_tiled_kernel<QKK_Q8_0>, grid, dim3(GT_THREADS), 0, st, W, X, Y, M, N, K); return true;
    case QKK_Q6_K: hipLaunchKernelGGL(gemm_tiled_kernel<QKK_Q6_K>, grid, dim3(GT_THREADS), 0, st, W, X, Y, M, N, K); return true;
    case QKK_IQ4_XS: hipLaunchKernelGGL(gemm_tiled_kernel<QKK_IQ4_XS>, grid, dim3(GT_THREADS), 0, st, W, X, Y, M, N, K); return true;
    case QKK_IQ3_XXS: hipLaunchKernelGGL(gemm_tiled_kernel<QKK_IQ3_XXS>, grid, dim3(GT_THREADS), 0, st, W, X, Y, M, N, K); return true;
    default: return false;
    }
}

} // namespace qk
