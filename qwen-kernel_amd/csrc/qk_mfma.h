// qk_mfma.h -- MFMA building blocks for the token-batched kernels.
//
// Orientation used throughout: A = activations (16 tokens x K), B = weights (K x 16 weight
// rows), so a lane's four outputs D[4*(l/16)+e][l%16] all belong to ONE weight row (l%16).
// The lane that decodes row l%16 for B therefore also owns that row's outputs, and per-block
// scales are applied lane-locally in fp32 AFTER the MFMA: the weight operand holds only the
// block's small integers (exact in half), the activation operand is split x = hi + lo (two
// halves, x exact to ~2^-22).  Kernels that fold a block's sub-scale into the weight operand (to
// make a lane's weight bytes contiguous) carry the rounding residual in a second operand.
#pragma once
#include "qk_device.h"

namespace qk {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

// K = 32 per instruction: lane l feeds A[l%16][8*(l/16)+e], B[8*(l/16)+e][l%16], e < 8.
__device__ __forceinline__ float4v mfma16x32(half8 a, half8 b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// K = 16 per instruction: lane l feeds A[l%16][4*(l/16)+e], B[4*(l/16)+e][l%16], e < 4.
__device__ __forceinline__ float4v mfma16x16(half4 a, half4 b, float4v c)
{
    return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
}

// Four unsigned bytes -> four halves (u - bias), exact: 0x6400 | u is the half 1024 + u.
__device__ __forceinline__ half4 bytes_to_half4(uint32_t u4, float bias)
{
    const uint32_t w01 = __builtin_amdgcn_perm(0x64646464u, u4, 0x04010400u); // bytes u0, 0x64, u1, 0x64
    const uint32_t w23 = __builtin_amdgcn_perm(0x64646464u, u4, 0x04030402u);
    const _Float16 b = (_Float16)(-(1024.f + bias));
    const half2v off = {b, b};
    const half2v lo = __builtin_bit_cast(half2v, w01) + off, hi = __builtin_bit_cast(half2v, w23) + off;
    return half4{lo[0], lo[1], hi[0], hi[1]};
}

// Activation rows staged in LDS in fragment order, so a wave's 64 lanes read 64 consecutive
// 8-byte (K=16 fragments) or 16-byte (K=32) pieces: no bank conflicts.
//   K=16 layout: [k/16][lane = 16*((k%16)/4) + token][k%4]
//   K=32 layout: [k/32][lane = 16*((k%32)/8) + token][k%8]
// Two planes (hi, lo) follow each other.  `stage_tokens` converts up to 16 fp32 rows
// (rows >= n_rows read as zero); row r of the tile is X + row_of(r)*K.
//   K: width of the staged tile; stride: floats between consecutive source rows.
template <int KF, typename RowOf>
__device__ __forceinline__ void stage_tokens(_Float16* __restrict__ s_hi, _Float16* __restrict__ s_lo,
                                             const float* __restrict__ X, uint32_t K, uint32_t stride,
                                             uint32_t n_rows, RowOf row_of, int tid, int nthreads)
{
    constexpr int PER = KF / 4; // elements a lane holds per fragment
    const uint32_t quads = 16u * K / 4; // float4 pieces in the tile
    for (uint32_t q = tid; q < quads; q += nthreads) {
        const uint32_t tok = q / (K / 4), k = (q % (K / 4)) * 4;
        float4 v = float4{0.f, 0.f, 0.f, 0.f};
        if (tok < n_rows) v = *(const float4*)(X + (size_t)row_of(tok) * stride + k);
        const float f[4] = {v.x, v.y, v.z, v.w};
        const uint32_t frag = k / KF, g = (k % KF) / PER, t0 = k % PER;
        const uint32_t off = ((frag * 4 + g) * 16 + tok) * PER + t0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const _Float16 hi = (_Float16)f[e];
            s_hi[off + e] = hi;
            s_lo[off + e] = (_Float16)(f[e] - (float)hi);
        }
    }
}

} // namespace qk
