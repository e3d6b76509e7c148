// qk_device.h -- device-side helpers shared by the gfx950 kernels: wave64 reductions
// on DPP, unaligned block-stream loads, half conversion, per-format lane tasks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qk_formats.h"

namespace qk {

constexpr int WAVE = 64;

// Two hooks that let a host-side build of these kernels (the tests' bounds and logic check; it
// defines both before this header is read) supply what only the device has:
// the dynamic LDS of a launch, declared at the top of a kernel, and the register constraint of the
// empty asm statements that pin values.
#ifndef QK_DYN_LDS
#define QK_DYN_LDS(type, name) extern __shared__ __attribute__((aligned(16))) type name[]
#endif
#ifndef QK_REG
#define QK_REG(x) "+v"(x)
#endif
// A third hook marks the table lookups in LDS (site = a small integer, the address and width of this
// lane's read): nothing on the device; the host-side build counts bank conflicts per wave instruction.
#ifndef QK_LDS_PROBE
#define QK_LDS_PROBE(site, ptr, bytes) ((void)0)
#endif
enum { QK_SITE_IQ3_GRID = 0, QK_SITE_IQ3_SIGN = 1, QK_SITE_IQ4_PAIR = 2, QK_SITE_IQ4_FLOAT = 3, QK_SITE_IQ3_GRID_WORD = 4 };

// ---- loads -----------------------------------------------------------------------
// GGUF blocks are 2-byte (Q8_0, Q6_K, IQ3_XXS) or 8-byte (IQ4_XS) aligned.  gfx950
// global loads accept any byte alignment, so a block field is fetched with the widest
// load that covers it; memcpy keeps the access well-defined for the compiler.
template <typename T>
__device__ __forceinline__ T ldg(const uint8_t* p)
{
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

__device__ __forceinline__ float h2f(uint16_t h)
{
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

template <int TYPE>
__host__ __device__ constexpr size_t qkk_row_bytes_dev(uint64_t k)
{
    return TYPE == 8 ? k / 32 * Q8_0_BYTES
         : TYPE == 14 ? k / 256 * Q6_K_BYTES
         : TYPE == 23 ? k / 256 * IQ4_XS_BYTES
         : TYPE == 18 ? k / 256 * IQ3_XXS_BYTES
         : TYPE == 1 ? k * 2 : k * 4;
}

// ---- publishing results to other workgroups of the same launch -----------------------------
// A release fence at device scope writes back the whole L2 of the XCD (buffer_wbl2); issued
// once per workgroup by a thousand workgroups it costs tens of microseconds.  Values another
// workgroup of the same launch will read are therefore stored with device-scope atomic stores
// (written through to memory); every lane that published waits for its own stores to be
// acknowledged (publish_wait) before the workgroup's barrier, the arrival is then counted with a
// relaxed device-scope atomic, and only the single workgroup that reads the values executes an
// acquire fence (cache invalidate).
__device__ __forceinline__ void publish(float* p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void publish(uint32_t* p, uint32_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Waits until every vector-memory operation of this wave, the publish() stores among them, has been
// acknowledged: s_waitcnt vmcnt(0) (expcnt and lgkmcnt fields left at their maxima).  A workgroup-scope
// release fence does not do this -- it only drains the LDS/scalar counter -- so without the wait the
// arrival below could be counted while a published value is still on its way to another L2 channel.
__device__ __forceinline__ void publish_wait()
{
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}
// Called by ONE thread after a __syncthreads() that follows the workgroup's publish() +
// publish_wait() calls (the caller's own stores are waited for here as well).  Returns true for the
// workgroup that arrives last; that one may then read what the others published.
__device__ __forceinline__ bool arrive_last(uint32_t* counter, uint32_t n_workgroups)
{
    publish_wait();
    const bool last =
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_workgroups - 1;
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}

// ---- wave64 reductions -------------------------------------------------------------
// Butterfly inside each row of 16 lanes on DPP (quad_perm xor1, xor2, row_half_mirror,
// row_mirror): after these four steps every lane of a row holds the row's sum.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
constexpr int DPP_XOR1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141; // lanes 0..7 reversed inside each 8
constexpr int DPP_MIRROR = 0x140;      // lanes 0..15 reversed inside each 16

// Sum over groups of N adjacent lanes (N = 4, 8 or 16); every lane gets its group's sum.
template <int N>
__device__ __forceinline__ float group_sum(float v)
{
    v += dpp_f<DPP_XOR1>(v);
    v += dpp_f<DPP_XOR2>(v);
    if (N >= 8) v += dpp_f<DPP_HALF_MIRROR>(v);
    if (N >= 16) v += dpp_f<DPP_MIRROR>(v);
    return v;
}

__device__ __forceinline__ float readlane_f(float v, int lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over the whole wave; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v = group_sum<16>(v);
    return (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
}

// Sum over groups of N adjacent lanes for N = 32 (two rows).
__device__ __forceinline__ float group_sum32(float v)
{
    v = group_sum<16>(v);
    // lanes 0..31 want rows 0+1, lanes 32..63 rows 2+3: swap rows with ds_swizzle-free DPP
    // row_shr is row-local, so fetch the partner row through bpermute.
    const int lane = (int)__lane_id();
    const float o = __builtin_bit_cast(
        float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, v)));
    return v + o;
}

template <int N>
__device__ __forceinline__ float lanes_sum(float v)
{
    if constexpr (N == 64) return wave_sum(v);
    else if constexpr (N == 32) return group_sum32(v);
    else return group_sum<N>(v);
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t v)
{
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t t = __shfl_up(v, d);
        if (lane >= d) v += t;
    }
    return v;
}

// Sum over a workgroup of four waves (256 threads, all of them calling) in wave order; every
// thread returns the same bits.  s_red: four floats of LDS.
__device__ __forceinline__ float block_sum4(float v, float* s_red)
{
    const float w = wave_sum(v);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = w;
    __syncthreads();
    return ((s_red[0] + s_red[1]) + s_red[2]) + s_red[3];
}

__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f<DPP_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f<DPP_MIRROR>(v));
    return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)),
                 fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v)
{
    int x = (int)v; // callers pass values < 2^31
    x = min(x, dpp_i<DPP_XOR1>(x));
    x = min(x, dpp_i<DPP_XOR2>(x));
    x = min(x, dpp_i<DPP_HALF_MIRROR>(x));
    x = min(x, dpp_i<DPP_MIRROR>(x));
    const int a = min(__builtin_amdgcn_readlane(x, 0), __builtin_amdgcn_readlane(x, 16));
    const int b = min(__builtin_amdgcn_readlane(x, 32), __builtin_amdgcn_readlane(x, 48));
    return (uint32_t)min(a, b);
}

// ---- per-format lane tasks -----------------------------------------------------------
// Every quantised format is cut so that ONE LANE owns 32 weights of a row per pass and a
// wave covers 2048 consecutive weights: Q8_0 one block per lane; IQ4_XS one 32-weight
// sub-block; IQ3_XXS one 32-weight group (8 grid bytes + its aux word); Q6_K four runs of
// 8 weights that share 8 qh bytes.  XS is the lane's slice of the activation row.

struct XSlice {
    float v[32];
};

// Where the lane's 32 activations live, as four runs of 8 floats: offset of run c.
template <int TYPE>
__device__ __forceinline__ int xrun_offset(int lane_in_row, int c)
{
    if constexpr (TYPE == 14) { // Q6_K: block = lane/8, half n = (lane%8)/4, l0 = 8*(lane%4)
        const int b = lane_in_row >> 3, n = (lane_in_row >> 2) & 1, l0 = (lane_in_row & 3) * 8;
        return b * 256 + n * 128 + c * 32 + l0;
    } else {
        return lane_in_row * 32 + c * 8;
    }
}

template <int TYPE>
__device__ __forceinline__ void load_xslice(XSlice& xs, const float* __restrict__ x, int lane_in_row)
{
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const float4* p = (const float4*)(x + xrun_offset<TYPE>(lane_in_row, c));
        const float4 a = p[0], b = p[1];
        xs.v[c * 8 + 0] = a.x; xs.v[c * 8 + 1] = a.y; xs.v[c * 8 + 2] = a.z; xs.v[c * 8 + 3] = a.w;
        xs.v[c * 8 + 4] = b.x; xs.v[c * 8 + 5] = b.y; xs.v[c * 8 + 6] = b.z; xs.v[c * 8 + 7] = b.w;
    }
}

// IQ3_XXS codebook in device memory (one copy per translation unit; 1 KiB).
static __device__ const uint32_t g_iq3xxs_grid[256] = {QK_IQ3XXS_GRID_ROWS};

// LDS tables used by the IQ formats.
struct IqTables {
    uint32_t grid[256];
    float iq4[16];
};

// IQ3_XXS tables for the packed-half dot product: the codebook as four half magnitudes per
// entry, and per 7-bit sign selector the sign bits of its eight weights in half positions
// (bit 15 / bit 31 of four dwords; the eighth sign is the parity of the seven).
struct Iq3HalfTables {
    uint2 grid[256];
    uint4 sign[128];
};
typedef _Float16 qk_half2 __attribute__((ext_vector_type(2)));

// Thread i < 256 fills entry i of the codebook (grid_word = codebook entry i as four bytes) and,
// for i < 128, sign entry i.
__device__ __forceinline__ void fill_iq3_half_entry(Iq3HalfTables& t, uint32_t i, uint32_t grid_word)
{
    const qk_half2 a = {(_Float16)(float)(grid_word & 255u), (_Float16)(float)((grid_word >> 8) & 255u)};
    const qk_half2 b = {(_Float16)(float)((grid_word >> 16) & 255u), (_Float16)(float)(grid_word >> 24)};
    t.grid[i] = uint2{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b)};
    if (i < 128) {
        const uint32_t s8 = i | ((__builtin_popcount(i) & 1u) << 7);
        uint32_t w[4];
#pragma unroll
        for (int p = 0; p < 4; p++) w[p] = (((s8 >> (2 * p)) & 1u) << 15) | (((s8 >> (2 * p + 1)) & 1u) << 31);
        t.sign[i] = uint4{w[0], w[1], w[2], w[3]};
    }
}

// A lane's 32 consecutive activations as 16 pairs of halves, value = hi + lo (exact to about
// 2^-22 of the value): the operands of v_dot2_f32_f16.
struct XSliceH {
    qk_half2 hi[16], lo[16];
};

__device__ __forceinline__ void split_xslice(XSliceH& h, const XSlice& xs)
{
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const _Float16 a = (_Float16)xs.v[2 * i], b = (_Float16)xs.v[2 * i + 1];
        h.hi[i] = qk_half2{a, b};
        h.lo[i] = qk_half2{(_Float16)(xs.v[2 * i] - (float)a), (_Float16)(xs.v[2 * i + 1] - (float)b)};
    }
}

// IQ4_XS codebook by byte: the weights j and j + 16 of a 32-weight sub-block share byte j, so entry b
// holds (kv[b & 15], kv[b >> 4]) as two halves (the codebook values are integers below 128: exact).
static __device__ const int8_t g_iq4nl[16] = {QK_IQ4NL_VALUES};
struct Iq4PairTable {
    uint32_t pair[256];
};
__device__ __forceinline__ void fill_iq4_pair_entry(Iq4PairTable& t, uint32_t i) // thread i < 256 fills entry i
{
    const qk_half2 v = {(_Float16)(float)g_iq4nl[i & 15u], (_Float16)(float)g_iq4nl[i >> 4]};
    t.pair[i] = __builtin_bit_cast(uint32_t, v);
}
// The activations paired the same way: pair j = (x[j], x[j + 16]), as hi + lo halves.
__device__ __forceinline__ void split_xslice_iq4(XSliceH& h, const XSlice& xs)
{
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const _Float16 a = (_Float16)xs.v[j], b = (_Float16)xs.v[j + 16];
        h.hi[j] = qk_half2{a, b};
        h.lo[j] = qk_half2{(_Float16)(xs.v[j] - (float)a), (_Float16)(xs.v[j + 16] - (float)b)};
    }
}

// Bytes of weights one lane fetches per pass, held in registers between the load and the
// arithmetic so several rows can be in flight.
template <int TYPE>
struct LaneW;

template <>
struct LaneW<8> { // Q8_0
    uint32_t q[8];
    uint16_t d;
    // Optimisation barrier: keeps the compiler from hoisting this row's decoded weights out
    // of a loop over activation rows (that would hold 32 floats per row in registers).
    __device__ __forceinline__ void touch()
    {
#pragma unroll
        for (int i = 0; i < 8; i++) asm volatile("" : QK_REG(q[i]));
    }
    __device__ __forceinline__ void load(const uint8_t* row, int lane_in_row)
    {
        const uint8_t* p = row + (size_t)lane_in_row * Q8_0_BYTES;
        d = ldg<uint16_t>(p);
        const uint4 a = ldg<uint4>(p + 2), b = ldg<uint4>(p + 18);
        q[0] = a.x; q[1] = a.y; q[2] = a.z; q[3] = a.w;
        q[4] = b.x; q[5] = b.y; q[6] = b.z; q[7] = b.w;
    }
    __device__ __forceinline__ float dot(const XSlice& xs, const float*, const IqTables*, int) const
    {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int j = 0; j < 4; j++) s += (float)(int8_t)(q[i] >> (8 * j)) * xs.v[i * 4 + j];
        }
        return h2f(d) * s;
    }
};

template <>
struct LaneW<14> { // Q6_K
    uint2 qa, qb, qh;
    uint32_t sc4; // the four sub-scales of this lane's runs, one per byte
    uint16_t d;
    __device__ __forceinline__ void touch()
    {
        asm volatile("" : QK_REG(qa.x), QK_REG(qa.y), QK_REG(qb.x), QK_REG(qb.y), QK_REG(qh.x), QK_REG(qh.y));
    }
    __device__ __forceinline__ void load(const uint8_t* row, int lane_in_row)
    {
        const int b = lane_in_row >> 3, n = (lane_in_row >> 2) & 1, l0 = (lane_in_row & 3) * 8;
        const uint8_t* p = row + (size_t)b * Q6_K_BYTES;
        qa = ldg<uint2>(p + 64 * n + l0);
        qb = ldg<uint2>(p + 64 * n + 32 + l0);
        qh = ldg<uint2>(p + Q6_K_QH + 32 * n + l0);
        // scales 8n + is + {0,2,4,6}, is = l0/16: fetch the 8 scales of this half
        const uint2 s8 = ldg<uint2>(p + Q6_K_SC + 8 * n);
        const int is = l0 >> 4;
        const uint32_t lo = is ? (s8.x >> 8) : s8.x, hi = is ? (s8.y >> 8) : s8.y;
        sc4 = (lo & 0xFFu) | ((lo >> 8) & 0xFF00u) | ((hi & 0xFFu) << 16) | ((hi << 8) & 0xFF000000u);
        d = ldg<uint16_t>(p + Q6_K_D);
    }
    // xsum[c] = sum of run c of the activations (the -32 offset is applied through it)
    __device__ __forceinline__ float dot(const XSlice& xs, const float* xsum, const IqTables*, int) const
    {
        float tot = 0.f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint2 ql = (c & 1) ? qb : qa;
            const int sh = 2 * c;
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const uint32_t l4 = w ? ql.y : ql.x, h4 = w ? qh.y : qh.x;
                const uint32_t nib = (c >= 2 ? (l4 >> 4) : l4) & 0x0F0F0F0Fu;
                const uint32_t q4 = nib | (((h4 >> sh) << 4) & 0x30303030u);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    s += (float)((q4 >> (8 * j)) & 0xFFu) * xs.v[c * 8 + w * 4 + j];
            }
            const float scv = (float)(int8_t)(sc4 >> (8 * c));
            tot += scv * (s - 32.f * xsum[c]);
        }
        return h2f(d) * tot;
    }
};

template <>
struct LaneW<23> { // IQ4_XS
    uint4 q;
    uint2 hdr; // d | scales_h<<16, scales_l[4]
    __device__ __forceinline__ void touch() { asm volatile("" : QK_REG(q.x), QK_REG(q.y), QK_REG(q.z), QK_REG(q.w)); }
    __device__ __forceinline__ void load(const uint8_t* row, int lane_in_row)
    {
        const int b = lane_in_row >> 3, ib = lane_in_row & 7;
        const uint8_t* p = row + (size_t)b * IQ4_XS_BYTES;
        hdr = ldg<uint2>(p);
        q = ldg<uint4>(p + IQ4_XS_QS + 16 * ib);
    }
    __device__ __forceinline__ float dot(const XSlice& xs, const float*, const IqTables* tab, int lane_in_row) const
    {
        const float* lut = tab->iq4; // the codebook as floats in LDS
        const int ib = lane_in_row & 7;
        const uint32_t sh = hdr.x >> 16;
        const int ls = (int)(((hdr.y >> (4 * ib)) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
        const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t byte = (qq[i] >> (8 * j)) & 0xFFu;
                QK_LDS_PROBE(QK_SITE_IQ4_FLOAT, &lut[byte & 15u], 4);
                s += lut[byte & 15u] * xs.v[i * 4 + j];
                QK_LDS_PROBE(QK_SITE_IQ4_FLOAT, &lut[byte >> 4], 4);
                s += lut[byte >> 4] * xs.v[16 + i * 4 + j];
            }
        }
        return h2f((uint16_t)hdr.x) * (float)ls * s;
    }
    // The same product on packed halves: one LDS lookup per byte gives both of its weights, each
    // v_dot2_f32_f16 takes them against a pair of activations (hi, then lo).  The sixteen lookups are
    // issued before the first product so that their latencies overlap.
    __device__ __forceinline__ float dot_h(const XSliceH& xh, const Iq4PairTable* tab, int lane_in_row) const
    {
        const int ib = lane_in_row & 7;
        const uint32_t sh = hdr.x >> 16;
        const int ls = (int)(((hdr.y >> (4 * ib)) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
        const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
        uint32_t w[16];
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const uint32_t* e = &tab->pair[(qq[k >> 2] >> (8 * (k & 3))) & 0xFFu];
            QK_LDS_PROBE(QK_SITE_IQ4_PAIR, e, 4);
            w[k] = *e;
        }
        __builtin_amdgcn_sched_barrier(0);
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const qk_half2 wk = __builtin_bit_cast(qk_half2, w[k]);
            s0 = __builtin_amdgcn_fdot2(wk, xh.hi[k], s0, false);
            s1 = __builtin_amdgcn_fdot2(wk, xh.lo[k], s1, false);
        }
        return h2f((uint16_t)hdr.x) * (float)ls * (s0 + s1);
    }
};

template <>
struct LaneW<18> { // IQ3_XXS
    uint2 g;      // 8 grid indices
    uint32_t aux; // 4 x 7-bit sign selectors + 4-bit scale
    uint16_t d;
    __device__ __forceinline__ void touch() { asm volatile("" : QK_REG(g.x), QK_REG(g.y), QK_REG(aux)); }
    __device__ __forceinline__ void load(const uint8_t* row, int lane_in_row)
    {
        const int b = lane_in_row >> 3, ib = lane_in_row & 7;
        const uint8_t* p = row + (size_t)b * IQ3_XXS_BYTES;
        d = ldg<uint16_t>(p);
        g = ldg<uint2>(p + IQ3_XXS_QS + 8 * ib);
        aux = ldg<uint32_t>(p + IQ3_XXS_AUX + 4 * ib);
    }
    __device__ __forceinline__ float dot(const XSlice& xs, const float*, const IqTables* tab, int) const
    {
        const uint32_t* grid = tab->grid; // 256 codewords in LDS
        float s = 0.f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t s7 = (aux >> (7 * l)) & 127u;
            const uint32_t sg = s7 | ((__builtin_popcount(s7) & 1u) << 7);
            const uint32_t gw = l < 2 ? g.x : g.y;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                QK_LDS_PROBE(QK_SITE_IQ3_GRID_WORD, &grid[(gw >> (16 * (l & 1) + 8 * hh)) & 0xFFu], 4);
                const uint32_t cw = grid[(gw >> (16 * (l & 1) + 8 * hh)) & 0xFFu];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float mag = (float)((cw >> (8 * j)) & 0xFFu);
                    const uint32_t neg = (sg << (31 - (4 * hh + j))) & 0x80000000u;
                    const float xv = __builtin_bit_cast(
                        float, __builtin_bit_cast(uint32_t, xs.v[l * 8 + hh * 4 + j]) ^ neg);
                    s += mag * xv;
                }
            }
        }
        return h2f(d) * (0.5f + (float)(aux >> 28)) * 0.5f * s;
    }
    // The same product on packed halves: signed magnitudes come out of two LDS lookups and two
    // XORs per four weights, each v_dot2_f32_f16 takes two weights (products exact, fp32 sums).  All
    // twelve lookups are issued before the first product, so that their latencies overlap (one at a
    // time, as the compiler had scheduled them, a lone lookup's latency was paid twelve times).
    // The product as the per-lane gate/up launch runs it (the form its device results and timings belong
    // to): lookups where they are used, the compiler's schedule.
    __device__ __forceinline__ float dot_h_inline(const XSliceH& xh, const Iq3HalfTables* tab) const
    {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint4 sm = tab->sign[(aux >> (7 * l)) & 127u];
            const uint32_t gw = l < 2 ? g.x : g.y;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                const uint2 m = tab->grid[(gw >> (16 * (l & 1) + 8 * hh)) & 0xFFu];
                const qk_half2 w01 = __builtin_bit_cast(qk_half2, m.x ^ (hh ? sm.z : sm.x));
                const qk_half2 w23 = __builtin_bit_cast(qk_half2, m.y ^ (hh ? sm.w : sm.y));
                const int q = l * 4 + hh * 2;
                s0 = __builtin_amdgcn_fdot2(w01, xh.hi[q], s0, false);
                s1 = __builtin_amdgcn_fdot2(w23, xh.hi[q + 1], s1, false);
                s0 = __builtin_amdgcn_fdot2(w01, xh.lo[q], s0, false);
                s1 = __builtin_amdgcn_fdot2(w23, xh.lo[q + 1], s1, false);
            }
        }
        return h2f(d) * (0.5f + (float)(aux >> 28)) * 0.5f * (s0 + s1);
    }
    __device__ __forceinline__ float dot_h(const XSliceH& xh, const Iq3HalfTables* tab) const
    {
        uint2 m[8];
        uint4 sg[4];
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint4* se = &tab->sign[(aux >> (7 * l)) & 127u];
            QK_LDS_PROBE(QK_SITE_IQ3_SIGN, se, 16);
            sg[l] = *se;
            const uint32_t gw = l < 2 ? g.x : g.y;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                const uint2* ge = &tab->grid[(gw >> (16 * (l & 1) + 8 * hh)) & 0xFFu];
                QK_LDS_PROBE(QK_SITE_IQ3_GRID, ge, 8);
                m[l * 2 + hh] = *ge;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                const qk_half2 w01 = __builtin_bit_cast(qk_half2, m[l * 2 + hh].x ^ (hh ? sg[l].z : sg[l].x));
                const qk_half2 w23 = __builtin_bit_cast(qk_half2, m[l * 2 + hh].y ^ (hh ? sg[l].w : sg[l].y));
                const int q = l * 4 + hh * 2;
                s0 = __builtin_amdgcn_fdot2(w01, xh.hi[q], s0, false);
                s1 = __builtin_amdgcn_fdot2(w23, xh.hi[q + 1], s1, false);
                s0 = __builtin_amdgcn_fdot2(w01, xh.lo[q], s0, false);
                s1 = __builtin_amdgcn_fdot2(w23, xh.lo[q + 1], s1, false);
            }
        }
        return h2f(d) * (0.5f + (float)(aux >> 28)) * 0.5f * (s0 + s1);
    }
};

__device__ __forceinline__ void fill_iq_tables(IqTables& t, const uint32_t* __restrict__ grid_g,
                                               int tid, int nthreads)
{
    constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
    for (int i = tid; i < 256; i += nthreads) t.grid[i] = grid_g[i];
    if (tid < 16) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) v = tid == i ? (float)kv[i] : v;
        t.iq4[tid] = v;
    }
}


} // namespace qk
