// qk_mfma.h -- MFMA building blocks for the token-batched kernels.
//
// Orientation used throughout: A = activations (16 rows x K), B = weights (K x 16 weight
// rows), so a lane's four outputs D[4*(l/16)+e][l%16] all belong to ONE weight row (l%16):
// the lane that decodes row l%16 for B also owns that row's outputs, and the row's fp16
// super-block scale is applied lane-locally in fp32 AFTER the MFMA.  The activation operand
// is split x = hi + lo (two halves, x exact to ~2^-22).  The weight operand holds the block's
// integers times the block's integer sub-scale; where that product does not fit a half the
// rounding residual goes into a second operand (one more MFMA), so weights are as exact.
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

} // namespace qk
