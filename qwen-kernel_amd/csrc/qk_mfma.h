// qk_mfma.h -- MFMA building blocks for the token-batched kernels.
//
// Orientation used throughout: A = activations (16 tokens x K), B = weights (K x 16 weight
// rows), so a lane's four outputs D[4*(l/16)+e][l%16] all belong to ONE weight row (l%16).
// The lane that decodes row l%16 for B therefore also owns that row's outputs, and per-block
// scales are applied lane-locally in fp32 AFTER the MFMA: the weight operand holds only the
// block's small integers (exact in half), the activation operand is split x = hi + lo (two
// halves, x exact to ~2^-22).  Kernels that fold a block's integer sub-scale into the weight
// operand (to make a lane's weight bytes contiguous) round that product to half once.
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

// Same LDS layouts as stage_tokens, written for speed: every thread converts whole lane
// pieces (KE = 8 halves for K=32 fragments, 4 for K=16), all global loads of a thread are in
// flight together, and consecutive threads write consecutive LDS pieces.  KT = staged width;
// up to 16 rows, rows >= n_rows read as zero; row r of the tile is X + row_of(r)*stride.
template <int KE, int KT, int NTHREADS, typename RowOf>
__device__ __forceinline__ void stage_rows(_Float16* __restrict__ s_hi, _Float16* __restrict__ s_lo,
                                           const float* __restrict__ X, uint32_t stride, uint32_t n_rows,
                                           RowOf row_of, int tid)
{
    constexpr int PIECES = 16 * KT / KE, IT = (PIECES + NTHREADS - 1) / NTHREADS;
    float v[IT][KE];
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const uint32_t q = min((uint32_t)(tid + it * NTHREADS), (uint32_t)PIECES - 1);
        const uint32_t row = q & 15u, g = (q >> 4) & 3u, step = q >> 6;
        const float* src = X + (size_t)row_of(min(row, n_rows - 1)) * stride + step * (4 * KE) + g * KE;
#pragma unroll
        for (int c = 0; c < KE / 4; c++) {
            const float4 f = *(const float4*)(src + 4 * c);
            v[it][4 * c] = f.x; v[it][4 * c + 1] = f.y; v[it][4 * c + 2] = f.z; v[it][4 * c + 3] = f.w;
        }
    }
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const uint32_t q = tid + it * NTHREADS;
        if (PIECES % NTHREADS != 0 && q >= (uint32_t)PIECES) break;
        const float keep = (q & 15u) < n_rows ? 1.f : 0.f;
        _Float16 hi[KE], lo[KE];
#pragma unroll
        for (int e = 0; e < KE; e++) {
            const float x = v[it][e] * keep;
            hi[e] = (_Float16)x;
            lo[e] = (_Float16)(x - (float)hi[e]);
        }
        if constexpr (KE == 8) {
            *(half8*)(s_hi + (size_t)q * 8) = half8{hi[0], hi[1], hi[2], hi[3], hi[4], hi[5], hi[6], hi[7]};
            *(half8*)(s_lo + (size_t)q * 8) = half8{lo[0], lo[1], lo[2], lo[3], lo[4], lo[5], lo[6], lo[7]};
        } else {
            *(half4*)(s_hi + (size_t)q * 4) = half4{hi[0], hi[1], hi[2], hi[3]};
            *(half4*)(s_lo + (size_t)q * 4) = half4{lo[0], lo[1], lo[2], lo[3]};
        }
    }
}

// Staging for fragments that span one 256-weight super-block (8 steps of K = 32) in which a
// lane group does not take every fourth run of 8 weights but a cut that makes its share of
// the weight bytes contiguous in the block:
//   LAYOUT 0: group g holds weights [64g, 64g+64), step i the eight at 64g + 8i
//   LAYOUT 1 (Q6_K): group g holds, of the 128-weight half g/2, the 16-weight scale groups of
//             parity g%2; step i the eight at 128(g/2) + 32(i/2) + 16(g%2) + 8(i%2)
// (the four lane groups of one MFMA then lie in different scale groups, so all scales below
// the super-block's are folded into the weight operand).  LDS order is
// [fragment][step][lane = 16g + row][8 halves]; KT = staged width, up to 16 rows, rows >=
// n_rows read as zero; row r of the tile is X + row_of(r)*stride.
template <int LAYOUT, int KT, int NTHREADS, typename RowOf>
__device__ __forceinline__ void stage_rows256(_Float16* __restrict__ s_hi, _Float16* __restrict__ s_lo,
                                              const float* __restrict__ X, uint32_t stride, uint32_t n_rows,
                                              RowOf row_of, int tid)
{
    constexpr int PIECES = 16 * KT / 8, IT = (PIECES + NTHREADS - 1) / NTHREADS;
    float4 v[IT][2];
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const uint32_t q = min((uint32_t)(tid + it * NTHREADS), (uint32_t)PIECES - 1);
        const uint32_t row = q & 15u, g = (q >> 4) & 3u, i = (q >> 6) & 7u, frag = q >> 9;
        const uint32_t k = frag * 256 + (LAYOUT == 0 ? 64 * g + 8 * i
                                                     : 128 * (g >> 1) + 32 * (i >> 1) + 16 * (g & 1) + 8 * (i & 1));
        const float* src = X + (size_t)row_of(min(row, n_rows - 1)) * stride + k;
        v[it][0] = *(const float4*)src;
        v[it][1] = *(const float4*)(src + 4);
    }
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const uint32_t q = tid + it * NTHREADS;
        if (PIECES % NTHREADS != 0 && q >= (uint32_t)PIECES) break;
        const float keep = (q & 15u) < n_rows ? 1.f : 0.f;
        const float f[8] = {v[it][0].x, v[it][0].y, v[it][0].z, v[it][0].w, v[it][1].x, v[it][1].y, v[it][1].z, v[it][1].w};
        half8 hi, lo;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x = f[e] * keep;
            hi[e] = (_Float16)x;
            lo[e] = (_Float16)(x - (float)hi[e]);
        }
        *(half8*)(s_hi + (size_t)q * 8) = hi;
        *(half8*)(s_lo + (size_t)q * 8) = lo;
    }
}

} // namespace qk
