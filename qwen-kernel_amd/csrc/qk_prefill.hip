// qk_prefill.hip -- batched-prefill kernels for gfx950: pair grouping and the Q8_0 dense
// projection GEMM (cooperative matrix-core stream for K = 256..2048 and N >= 8, a lane-direct
// MFMA kernel otherwise); the grouped-expert MoE entry point forwards to the expert-major
// kernels of qk_moe_grouped.hip / qk_moe_mfma.hip.
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {

// Counting sort of (token, pick) pairs by expert in one workgroup.  Pairs inside an expert
// come out in ascending (token, pick) order: each thread owns a contiguous run of pairs, a
// prefix sum over per-thread counts replaces the reference's LDS atomics
// (reference shaders/moe_group_pairs.comp:29,48), so the output is deterministic.
__global__ __launch_bounds__(1024) void group_pairs_kernel(const qkk_sel* __restrict__ sel,
                                                           uint32_t n_tokens, uint32_t E, uint32_t k,
                                                           uint32_t* __restrict__ offsets,
                                                           uint32_t* __restrict__ pairs)
{
    __shared__ uint32_t s_count[QKK_MAX_EXPERTS + 1];
    __shared__ uint32_t s_base[QKK_MAX_EXPERTS + 1];
    const uint32_t np = n_tokens * k;
    for (uint32_t e = threadIdx.x; e <= E; e += blockDim.x) s_count[e] = 0;
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < np; p += blockDim.x)
        atomicAdd(&s_count[min(sel[p / k].ids[p % k], E - 1)], 1u);
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t off = 0;
        for (uint32_t e = 0; e < E; e++) {
            s_base[e] = off;
            off += s_count[e];
        }
        s_base[E] = off;
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = s_base[e];
    // one thread per expert walks the pairs in order: E <= 512 threads busy, np*E/blockDim
    // comparisons each -- small next to the GEMMs it feeds, and order-stable
    for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) {
        if (s_count[e] == 0) continue;
        uint32_t dst = s_base[e];
        for (uint32_t p = 0; p < np; p++)
            if (min(sel[p / k].ids[p % k], E - 1) == e) pairs[dst++] = ((p / k) << 4) | (p % k);
    }
}


// ---- MFMA building blocks -------------------------------------------------------------------
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

// v_mfma_f32_16x16x32_f16: lane l feeds A[l%16][8*(l/16)+e] and B[8*(l/16)+e][l%16], e < 8,
// and receives D[4*(l/16)+e][l%16], e < 4.
__device__ __forceinline__ float4v mfma16(half8 a, half8 b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Eight int8 weights (two dwords) times the block scale -> eight halves.  Each byte q becomes
// the half 1024 + (q + 128) by pasting it under the exponent 0x64, then -1152 gives q exactly
// and one rounded multiply by d gives half(d*q): the same value as converting the fp32
// product d*q to half (the product is exact in fp32), which is what the reference stages
// (reference shaders/gemm_q8_0_coopmat2.comp:60-106).
__device__ __forceinline__ half8 q8_to_half8(uint32_t q0, uint32_t q1, _Float16 d)
{
    const uint32_t u0 = q0 ^ 0x80808080u, u1 = q1 ^ 0x80808080u;
    uint32_t w[4];
    w[0] = 0x64006400u | (u0 & 0xFFu) | ((u0 & 0xFF00u) << 8);
    w[1] = 0x64006400u | ((u0 >> 16) & 0xFFu) | ((u0 >> 8) & 0xFF0000u);
    w[2] = 0x64006400u | (u1 & 0xFFu) | ((u1 & 0xFF00u) << 8);
    w[3] = 0x64006400u | ((u1 >> 16) & 0xFFu) | ((u1 >> 8) & 0xFF0000u);
    const half2v off = {(_Float16)-1152.f, (_Float16)-1152.f}, dd = {d, d};
    half8 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const half2v v = (__builtin_bit_cast(half2v, w[i]) + off) * dd;
        r[2 * i] = v[0];
        r[2 * i + 1] = v[1];
    }
    return r;
}

// ---- dense Q8_0 projection -------------------------------------------------------------------
// Workgroup tile: 64 weight rows x 16*NT tokens, four waves as 2 (row halves) x 2 (token
// halves); a wave owns two 16-row tiles and NT/2 token tiles, so every activation fragment it
// reads from LDS feeds two MFMAs.  Per K step of 32 (one Q8_0 block per row) a lane fetches
// its 8 weights straight from the block stream in the MFMA A layout -- weights never pass
// through LDS -- while the activation tile [16*NT tokens][32] is split into half hi + half lo
// (x = hi + lo to ~2^-22; SPLIT=false keeps hi only, the reference's single-f16 staging) and
// staged in LDS for all four waves.  Global loads run D steps ahead of the MFMAs in registers.
template <int NT, bool SPLIT, int D>
__global__ __launch_bounds__(256) void gemm_q8_0_kernel(const uint8_t* __restrict__ W,
                                                        const float* __restrict__ X, float* __restrict__ Y,
                                                        uint32_t M, uint32_t K, uint32_t N)
{
    constexpr int BN = 16 * NT, NTW = NT / 2; // D: steps of look-ahead; K/32 must be a multiple of D
    constexpr int FPT = BN * 32 / 256; // floats of the activation tile staged per thread (4..16)
    __shared__ __attribute__((aligned(16))) _Float16 sX[2][2][BN][32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, g = lane >> 4, wm = wave & 1, wn = wave >> 1;
    const uint32_t row_bytes = K / 32 * Q8_0_BYTES;
    const uint32_t m_base = blockIdx.x * 64 + wm * 32;
    const uint32_t n0 = blockIdx.y * BN;
    const uint8_t* wrow[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++) wrow[mt] = W + (size_t)min(m_base + 16 * mt + i, M - 1) * row_bytes;
    const int xn = tid * FPT / 32, xk = tid * FPT % 32;
    const float* xsrc = X + (size_t)min(n0 + xn, N - 1) * K + xk;
    const uint32_t steps = K / 32;

    float4v acc[2][NTW];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int t = 0; t < NTW; t++) acc[mt][t] = float4v{0.f, 0.f, 0.f, 0.f};

    uint2 aq[D][2];
    uint32_t ad[D][2]; // dword holding the block scale in its low half (a full-register load)
    float xr[D][FPT];
    auto fetch = [&](int slot, uint32_t ks) {
#pragma unroll
        for (int mt = 0; mt < 2; mt++) {
            const uint8_t* p = wrow[mt] + (size_t)ks * Q8_0_BYTES;
            aq[slot][mt] = ldg<uint2>(p + 2 + 8 * g);
            ad[slot][mt] = ldg<uint32_t>(p);
        }
#pragma unroll
        for (int e = 0; e < FPT; e += 4) *(float4*)&xr[slot][e] = *(const float4*)(xsrc + (size_t)ks * 32 + e);
    };
#pragma unroll
    for (int j = 0; j < D; j++) fetch(j, j);

    // no branches inside the loop: the look-ahead fetch past the end re-reads the last step,
    // so the compiler can count outstanding loads exactly instead of draining them every step
    int buf = 0;
    for (uint32_t ks0 = 0; ks0 < steps; ks0 += D) {
#pragma unroll
        for (int j = 0; j < D; j++) {
            const uint32_t ks = ks0 + j;
#pragma unroll
            for (int e = 0; e < FPT; e++) {
                const _Float16 hi = (_Float16)xr[j][e];
                sX[buf][0][xn][xk + e] = hi;
                if (SPLIT) sX[buf][1][xn][xk + e] = (_Float16)(xr[j][e] - (float)hi);
            }
            half8 a[2];
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
                a[mt] = q8_to_half8(aq[j][mt].x, aq[j][mt].y, __builtin_bit_cast(_Float16, (uint16_t)ad[j][mt]));
            __syncthreads();
            fetch(j, min(ks + D, steps - 1));
#pragma unroll
            for (int t = 0; t < NTW; t++) {
                const int T = wn * NTW + t;
                const half8 bh = *(const half8*)&sX[buf][0][16 * T + i][8 * g];
#pragma unroll
                for (int mt = 0; mt < 2; mt++) acc[mt][t] = mfma16(a[mt], bh, acc[mt][t]);
                if (SPLIT) {
                    const half8 bl = *(const half8*)&sX[buf][1][16 * T + i][8 * g];
#pragma unroll
                    for (int mt = 0; mt < 2; mt++) acc[mt][t] = mfma16(a[mt], bl, acc[mt][t]);
                }
            }
            buf ^= 1;
        }
    }
    // D[4g+e][i]: rows are weight rows (m), columns tokens (n)
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
        const uint32_t m = m_base + 16 * mt + 4 * g;
#pragma unroll
        for (int t = 0; t < NTW; t++) {
            const uint32_t n = n0 + 16 * (wn * NTW + t) + i;
            if (n >= N) continue;
            float* dst = Y + (size_t)n * M + m;
            if (m + 3 < M && (M & 3u) == 0)
                *(float4*)dst = float4{acc[mt][t][0], acc[mt][t][1], acc[mt][t][2], acc[mt][t][3]};
            else
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (m + e < M) dst[e] = acc[mt][t][e];
        }
    }
}

// Cooperative matrix-core GEMM for K = 256..2048 (qk_gemm_coop.hip); false if the shape is not covered.
bool coop_gemm_launch(int type, const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N,
                      hipStream_t st);

} // namespace qk

using namespace qk;

extern "C" {

int qkk_moe_group_pairs(const qkk_sel* sel, uint32_t n_tokens, uint32_t n_expert, uint32_t n_used,
                        uint32_t* offsets, uint32_t* pairs, void* stream)
{
    if (!sel || !offsets || !pairs) return fail(QKK_EINVAL, "qkk_moe_group_pairs: null pointer");
    if (n_expert < 1 || n_expert > QKK_MAX_EXPERTS || n_used < 1 || n_used > QKK_MAX_USED)
        return fail(QKK_ESHAPE, "qkk_moe_group_pairs: n_expert %u / n_used %u out of range", n_expert, n_used);
    if (n_tokens == 0 || n_tokens > (1u << 28) / 16)
        return fail(QKK_ESHAPE, "qkk_moe_group_pairs: n_tokens %u out of range", n_tokens);
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(1024), 0, as_stream(stream), sel, n_tokens, n_expert,
                       n_used, offsets, pairs);
    return check_launch("qkk_moe_group_pairs");
}

int qkk_gemm_q8_0(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N, void* stream)
{
    if (!W || !X || !Y) return fail(QKK_EINVAL, "qkk_gemm_q8_0: null pointer");
    if (M == 0 || K == 0 || N == 0) return fail(QKK_EINVAL, "qkk_gemm_q8_0: M, K and N must be positive");
    if (K % 32) return fail(QKK_ESHAPE, "qkk_gemm_q8_0: K=%u is not a multiple of 32", K);
    if (!aligned16(W) || !aligned16(X) || !aligned16(Y))
        return fail(QKK_EINVAL, "qkk_gemm_q8_0: W, X and Y must be 16-byte aligned");
    if ((uint64_t)(N + 127) / 128 > 65535) return fail(QKK_ESHAPE, "qkk_gemm_q8_0: N=%u too large", N);
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    const uint8_t* w = (const uint8_t*)W;
    if (N >= 8 && coop_gemm_launch(QKK_Q8_0, w, X, Y, M, K, N, st)) return check_launch("qkk_gemm_q8_0");
    const uint32_t mb = (M + 63) / 64;
    const bool deep = (K / 32) % 4 == 0;
#define QK_GEMM_LAUNCH(NT_, D_, GY_)                                                                         \
    hipLaunchKernelGGL((gemm_q8_0_kernel<NT_, true, D_>), dim3(mb, GY_), dim3(256), 0, st, w, X, Y, M, K, N)
    // 64 tokens per workgroup measured fastest at N = 128 (twice the workgroups of the 128-token
    // tile: the K loop is latency-bound per workgroup, so more of them in flight wins)
    const int nt = N > 32 ? 4 : 2;
    const uint32_t gy = (N + 16 * nt - 1) / (16 * nt);
    if (nt == 4) { if (deep) QK_GEMM_LAUNCH(4, 4, gy); else QK_GEMM_LAUNCH(4, 1, gy); }
    else { if (deep) QK_GEMM_LAUNCH(2, 4, gy); else QK_GEMM_LAUNCH(2, 1, gy); }
#undef QK_GEMM_LAUNCH
    return check_launch("qkk_gemm_q8_0");
}
size_t qkk_moe_prefill_workspace_bytes(const qkk_moe_layer* L, uint32_t n_tokens)
{
    return qkk_moe_workspace_bytes(L, n_tokens);
}
int qkk_moe_prefill(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                    size_t workspace_bytes, uint32_t n_tokens, void* stream)
{
    return qkk_moe_decode(L, X, Y, sel, workspace, workspace_bytes, n_tokens, stream);
}

} // extern "C"
