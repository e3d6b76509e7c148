// qk_stream.h -- streaming block rows through a wave-private LDS area.
//
// The block formats pack fields at 2-byte alignment (34 / 98 / 210-byte blocks), so a lane that
// fetches its own block's fields from global memory issues several narrow, misaligned loads, and
// the address unit of the CU, which handles about one lane access per clock, becomes the limit long
// before the memory system does.  Here a wave copies the contiguous byte range of its rows with
// 16-byte loads -- consecutive lanes, consecutive 16-byte pieces: every cache line crosses the L1
// once, as full-width requests -- stores the pieces to an LDS area of its own (no workgroup barrier:
// LDS operations of one wave execute in order), and each lane then picks its block's fields out of
// LDS as aligned dwords plus v_alignbyte.  The loads of the next range are issued before the
// arithmetic of the current one, so the bytes in flight live in registers, not in occupancy.
#pragma once
#include "qk_device.h"
#include "qk_host.h"

namespace qk {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// The staging area is written as 16-byte pieces and read back as dwords and halfwords of the block
// fields: every access goes through a may_alias type, or type-based alias analysis lets the compiler
// move a later write of the area in front of reads of other types (it did).
typedef u32x4 u32x4_a __attribute__((may_alias));
typedef uint32_t u32_a __attribute__((may_alias));
typedef uint16_t u16_a __attribute__((may_alias));

// NP 16-byte pieces per lane: pieces lane, lane + 64, ... of a range of n pieces.  The LDS area holds
// NP * 1024 bytes: every lane stores every piece, so there is no branch on either side; lanes past
// the end of the range re-read its last piece (a line that is on its way anyway) and store it behind
// the range, where nothing reads it.
template <int NP>
struct WaveStage {
    static constexpr uint32_t AREA = NP * 1024u; // bytes of LDS per wave
    u32x4 r[NP];
    // g: 16-byte aligned start of the range of n >= 1 pieces
    __device__ __forceinline__ void fetch(const uint8_t* __restrict__ g, uint32_t n, int lane)
    {
        const u32x4_a* p = (const u32x4_a*)g;
#pragma unroll
        for (int j = 0; j < NP; j++) r[j] = p[min((uint32_t)(lane + 64 * j), n - 1)];
    }
    // The same with the address of every piece given by the caller: addr(i) for piece i = lane,
    // lane + 64, ... (ranges made of several runs, e.g. the same rows of several experts).  addr must
    // be valid for every i < 64 * NP.
    template <class F>
    __device__ __forceinline__ void fetch_at(F addr, int lane)
    {
#pragma unroll
        for (int j = 0; j < NP; j++) r[j] = *(const u32x4_a*)addr((uint32_t)(lane + 64 * j));
    }
    // The area belongs to the wave: the wave barriers (no instruction on the device, where the lanes
    // of a wave execute an LDS operation together and the operations in order) mark that the field
    // reads of the previous range come before these stores, and these stores before the next reads.
    __device__ __forceinline__ void commit(uint8_t* lds, int lane) const
    {
        u32x4_a* p = (u32x4_a*)lds;
        // wavefront-scope fences emit no instruction; they keep the compiler from moving the other
        // lanes' field reads across the stores (the barrier intrinsic alone orders execution, not memory)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int j = 0; j < NP; j++) p[lane + 64 * j] = r[j];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
};

// All vector-memory operations of the wave have completed.  Placed in front of a streaming loop so
// that values loaded before it (the activations) are not waited for inside it: the counter is in
// order, and a wait for an old load behind a new one would also wait for the loads of the next range.
__device__ __forceinline__ void vmem_drain()
{
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0), expcnt and lgkmcnt at their maxima
}

// 32 bits at byte offset `off` (a multiple of 4) of an LDS area whose base is 4-byte aligned.
__device__ __forceinline__ uint32_t lds_dw(const uint8_t* base, uint32_t off)
{
    return *(const u32_a*)(base + off);
}
// 64 bits at byte offset `off` (any multiple of 2): three aligned dwords, two funnel shifts.
__device__ __forceinline__ uint2 lds_u64_at(const uint8_t* base, uint32_t off)
{
    const uint32_t sh = off & 3u, o4 = off & ~3u;
    const uint32_t a = lds_dw(base, o4), c = lds_dw(base, o4 + 4), e = lds_dw(base, o4 + 8);
    return uint2{__builtin_amdgcn_alignbyte(c, a, sh), __builtin_amdgcn_alignbyte(e, c, sh)};
}
__device__ __forceinline__ uint32_t lds_u32_at(const uint8_t* base, uint32_t off)
{
    const uint32_t sh = off & 3u, o4 = off & ~3u;
    return __builtin_amdgcn_alignbyte(lds_dw(base, o4 + 4), lds_dw(base, o4), sh);
}
__device__ __forceinline__ uint16_t lds_u16_at(const uint8_t* base, uint32_t off)
{
    return *(const u16_a*)(base + off);
}

// Field readers: the lane's part of a row that lies in LDS at byte offset `row` (a multiple of 2) of
// an area whose base is 16-byte aligned -- the same fields LaneW<TYPE>::load takes from global
// memory.  They read up to 10 bytes past the fields, so an area keeps 16 spare bytes behind its
// last row.
template <int TYPE>
__device__ __forceinline__ void lane_load_lds(LaneW<TYPE>& w, const uint8_t* base, uint32_t row, int lane_in_row);

template <>
__device__ __forceinline__ void lane_load_lds<QKK_Q8_0>(LaneW<QKK_Q8_0>& w, const uint8_t* base, uint32_t row, int lir)
{
    const uint32_t B = row + (uint32_t)lir * Q8_0_BYTES, Q = B + 2, sh = Q & 3u, Q4 = Q & ~3u;
    uint32_t dw[9];
#pragma unroll
    for (int i = 0; i < 9; i++) dw[i] = lds_dw(base, Q4 + 4 * i);
#pragma unroll
    for (int i = 0; i < 8; i++) w.q[i] = __builtin_amdgcn_alignbyte(dw[i + 1], dw[i], sh);
    w.d = lds_u16_at(base, B);
}

template <>
__device__ __forceinline__ void lane_load_lds<QKK_IQ3_XXS>(LaneW<QKK_IQ3_XXS>& w, const uint8_t* base, uint32_t row, int lir)
{
    const uint32_t b = lir >> 3, ib = lir & 7;
    const uint32_t B = row + b * IQ3_XXS_BYTES;
    w.g = lds_u64_at(base, B + IQ3_XXS_QS + 8 * ib);
    w.aux = lds_u32_at(base, B + IQ3_XXS_AUX + 4 * ib);
    w.d = lds_u16_at(base, B);
}

template <>
__device__ __forceinline__ void lane_load_lds<QKK_IQ4_XS>(LaneW<QKK_IQ4_XS>& w, const uint8_t* base, uint32_t row, int lir)
{
    const uint32_t b = lir >> 3, ib = lir & 7;
    const uint32_t B = row + b * IQ4_XS_BYTES; // blocks are multiples of 8 bytes: with row a multiple of 4, aligned dwords
    w.hdr = uint2{lds_dw(base, B), lds_dw(base, B + 4)};
    const uint32_t Q = B + IQ4_XS_QS + 16 * ib;
    w.q = uint4{lds_dw(base, Q), lds_dw(base, Q + 4), lds_dw(base, Q + 8), lds_dw(base, Q + 12)};
}

template <>
__device__ __forceinline__ void lane_load_lds<QKK_Q6_K>(LaneW<QKK_Q6_K>& w, const uint8_t* base, uint32_t row, int lir)
{
    const uint32_t b = lir >> 3, n = (lir >> 2) & 1, l0 = (lir & 3) * 8;
    const uint32_t B = row + b * Q6_K_BYTES;
    w.qa = lds_u64_at(base, B + 64 * n + l0);
    w.qb = lds_u64_at(base, B + 64 * n + 32 + l0);
    w.qh = lds_u64_at(base, B + Q6_K_QH + 32 * n + l0);
    const uint2 s8 = lds_u64_at(base, B + Q6_K_SC + 8 * n);
    const int is = l0 >> 4;
    const uint32_t lo = is ? (s8.x >> 8) : s8.x, hi = is ? (s8.y >> 8) : s8.y;
    w.sc4 = (lo & 0xFFu) | ((lo >> 8) & 0xFF00u) | ((hi & 0xFFu) << 16) | ((hi << 8) & 0xFF000000u);
    w.d = lds_u16_at(base, B + Q6_K_D);
}

} // namespace qk
