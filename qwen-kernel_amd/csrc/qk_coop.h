// qk_coop.h -- cooperative weight streaming for the token-batched matrix-core kernels (the
// expert-major MoE projections and the batched LM head).
//
// The weight rows a workgroup works on are ONE contiguous byte range of a row-major tensor, so
// the workgroup copies it to LDS in double-buffered batches with coalesced 16-byte loads (the
// L1 sees every line once; per-lane loads of 16 different rows per wave were bound by the
// number of L1 accesses).  The eight waves split K: each keeps its 256-wide slice of the 16
// activation rows in registers as hi + lo half operands, decodes its fragments from LDS into
// v_mfma_f32_16x16x32_f16 weight operands, and the partial 16x16 results are summed through
// LDS in a fixed order (bit-reproducible).  Orientation and exactness: see qk_mfma.h.
#pragma once
#include "qk_host.h"
#include "qk_mfma.h"

namespace qk {

struct MfmaTables {
    uint32_t grid[256]; // IQ3_XXS codewords, four magnitudes per dword
    uint2 sign[128];    // IQ3_XXS sign selector -> 0xFF in the bytes of the eight weights to negate
    uint32_t iq4[4];    // IQ4 codebook, sixteen int8 in four dwords
};

__device__ static void fill_mfma_tables(MfmaTables& t, int tid, int nthreads)
{
    for (int i = tid; i < 256; i += nthreads) t.grid[i] = g_iq3xxs_grid[i];
    for (int i = tid; i < 128; i += nthreads) {
        const uint32_t s8 = (uint32_t)i | ((__builtin_popcount(i) & 1u) << 7); // eighth sign = parity
        const uint32_t a = ((s8 & 15u) * 0x00204081u) & 0x01010101u, b = ((s8 >> 4) * 0x00204081u) & 0x01010101u;
        t.sign[i] = uint2{(a << 8) - a, (b << 8) - b};
    }
    if (tid < 4) {
        constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (i / 4 == tid) w |= (uint32_t)(uint8_t)kv[i] << (8 * (i % 4));
        t.iq4[tid] = w;
    }
}

// Only what BFrag<TYPE> reads: the IQ3_XXS grid and signs, the IQ4_XS codebook, nothing for the others.
template <int TYPE>
__device__ static void fill_mfma_tables_for(MfmaTables& t, int tid, int nthreads)
{
    if constexpr (TYPE == QKK_IQ3_XXS) {
        for (int i = tid; i < 256; i += nthreads) t.grid[i] = g_iq3xxs_grid[i];
        for (int i = tid; i < 128; i += nthreads) {
            const uint32_t s8 = (uint32_t)i | ((__builtin_popcount(i) & 1u) << 7);
            const uint32_t a = ((s8 & 15u) * 0x00204081u) & 0x01010101u, b = ((s8 >> 4) * 0x00204081u) & 0x01010101u;
            t.sign[i] = uint2{(a << 8) - a, (b << 8) - b};
        }
    } else if constexpr (TYPE == QKK_IQ4_XS) {
        if (tid < 4) {
            constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 16; i++)
                if (i / 4 == tid) w |= (uint32_t)(uint8_t)kv[i] << (8 * (i % 4));
            t.iq4[tid] = w;
        }
    }
}

// ---- a lane's share of one 256-weight fragment of row (l%16), in the B-operand cut -----------------
// Lane group g = l/16 owns 64 of the fragment's 256 weights, chosen so that its bytes are
// CONTIGUOUS in the block and a fragment is two or three wide (LDS) reads:
//   LAYOUT 0: weights [64g, 64g+64), step i the eight at 64g + 8i
//   LAYOUT 1 (Q6_K): of the 128-weight half g/2 the 16-weight scale groups of parity g%2;
//             step i the eight at 128(g/2) + 32(i/2) + 16(g%2) + 8(i%2)
// Step i of 8 feeds eight of them to one K = 32 MFMA.  The four lane groups of a step
// then lie in different sub-blocks, so step(i, g, tab, lo) returns the weights times the
// sub-block scale as halves; post() is what remains, one fp32 factor per row and fragment,
// applied to the MFMA result.  Where that product does not fit a half exactly (SPLIT), `lo`
// receives the rounding residual (exact, by fma) and a third MFMA adds activations * lo, so
// the weights stay exact to ~2^-22 like the activations.
template <int TYPE>
struct BFrag;

__device__ __forceinline__ half8 scale8(half4 a, half4 b, _Float16 m)
{
    return half8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]} * m;
}
__device__ __forceinline__ half8 scale8(half4 a, half4 b, _Float16 m, half8& lo)
{
    const half8 v = half8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    const half8 mm = half8{m, m, m, m, m, m, m, m};
    const half8 hi = v * mm;
    lo = __builtin_elementwise_fma(v, mm, -hi);
    return hi;
}

template <>
struct BFrag<QKK_Q8_0> { // eight Q8_0 blocks; group g owns blocks 2g, 2g+1; d folded into the operand
    static constexpr int BYTES = 8 * Q8_0_BYTES, LAYOUT = 0;
    static constexpr bool SPLIT = true;
    uint4 q[4];
    uint32_t d[2]; // one register each: packing two halves would put ALU, and a wait, behind the loads
    __device__ __forceinline__ void load(const uint8_t* row, uint32_t fi, int g)
    {
        const uint8_t* b = row + (size_t)fi * BYTES + 2 * g * Q8_0_BYTES;
        d[0] = ldg<uint16_t>(b);
        q[0] = ldg<uint4>(b + 2);
        q[1] = ldg<uint4>(b + 18);
        d[1] = ldg<uint16_t>(b + Q8_0_BYTES);
        q[2] = ldg<uint4>(b + Q8_0_BYTES + 2);
        q[3] = ldg<uint4>(b + Q8_0_BYTES + 18);
    }
    __device__ __forceinline__ float post() const { return 1.f; }
    __device__ __forceinline__ half8 step(int i, int, const MfmaTables&, half8& lo) const
    {
        const uint4 v = q[i >> 1];
        const half4 a = bytes_to_half4(((i & 1) ? v.z : v.x) ^ 0x80808080u, 128.f);
        const half4 b = bytes_to_half4(((i & 1) ? v.w : v.y) ^ 0x80808080u, 128.f);
        return scale8(a, b, __builtin_bit_cast(_Float16, (uint16_t)d[i >> 2]), lo);
    }
};

template <>
struct BFrag<QKK_IQ3_XXS> { // group g owns sub-blocks 2g, 2g+1: 16 grid indices + 2 aux words
    static constexpr int BYTES = IQ3_XXS_BYTES, LAYOUT = 0;
    static constexpr bool SPLIT = false; // magnitude <= 62 times 2s+1 <= 31: exact in half
    uint4 idx;
    uint2 aux;
    uint16_t d;
    __device__ __forceinline__ void load(const uint8_t* row, uint32_t fi, int g)
    {
        const uint8_t* p = row + (size_t)fi * BYTES;
        d = ldg<uint16_t>(p);
        idx = ldg<uint4>(p + IQ3_XXS_QS + 16 * g);
        aux = ldg<uint2>(p + IQ3_XXS_AUX + 8 * g);
    }
    __device__ __forceinline__ float post() const { return h2f(d) * 0.25f; } // d * (2s+1)/4, 2s+1 in the operand
    // four magnitudes (bytes of cw, each <= 62), m = 0xFF in the bytes to negate -> four halves
    // +-mag, exact: the byte 0x80 +- mag under the exponent byte 0x64 is the half 1152 +- mag
    __device__ __forceinline__ static half4 signed4(uint32_t cw, uint32_t m)
    {
        const uint32_t pos = cw + 0x80808080u, neg = 0x80808080u - cw; // no carry between bytes
        return bytes_to_half4((neg & m) | (pos & ~m), 128.f);
    }
    __device__ __forceinline__ half8 step(int i, int, const MfmaTables& tab, half8&) const
    {
        const uint32_t a = (i >> 2) ? aux.y : aux.x;
        const uint2 m = tab.sign[(a >> (7 * (i & 3))) & 127u];
        const uint32_t w = (i >> 1) == 0 ? idx.x : (i >> 1) == 1 ? idx.y : (i >> 1) == 2 ? idx.z : idx.w;
        const uint32_t pr = w >> (16 * (i & 1));
        const half4 lo = signed4(tab.grid[pr & 255u], m.x), hi = signed4(tab.grid[(pr >> 8) & 255u], m.y);
        return scale8(lo, hi, (_Float16)(float)((a >> 27) | 1u));
    }
};

template <>
struct BFrag<QKK_IQ4_XS> { // group g owns sub-blocks 2g, 2g+1: 32 bytes of nibbles
    static constexpr int BYTES = IQ4_XS_BYTES, LAYOUT = 0;
    static constexpr bool SPLIT = true; // |codebook| <= 127 times |ls-32| <= 32
    uint4 q[2];
    uint2 hdr; // d | scales_h << 16, scales_l[4]
    __device__ __forceinline__ void load(const uint8_t* row, uint32_t fi, int g)
    {
        const uint8_t* p = row + (size_t)fi * BYTES;
        hdr = ldg<uint2>(p);
        q[0] = ldg<uint4>(p + IQ4_XS_QS + 32 * g);
        q[1] = ldg<uint4>(p + IQ4_XS_QS + 32 * g + 16);
    }
    __device__ __forceinline__ float post() const { return h2f((uint16_t)hdr.x); }
    // four nibbles (one per byte of n4, values 0..15) -> four codebook int8 -> four halves
    __device__ __forceinline__ static half4 lut4(uint32_t n4, const MfmaTables& tab)
    {
        const uint32_t sel = n4 & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(tab.iq4[1], tab.iq4[0], sel);
        const uint32_t hi = __builtin_amdgcn_perm(tab.iq4[3], tab.iq4[2], sel);
        const uint32_t t = (n4 >> 3) & 0x01010101u, m = (t << 8) - t;
        const uint32_t v = (hi & m) | (lo & ~m);
        return bytes_to_half4(v ^ 0x80808080u, 128.f);
    }
    __device__ __forceinline__ half8 step(int i, int g, const MfmaTables& tab, half8& lo) const
    {
        // sub-block 2g + i/4; within it weights 8t..8t+7 (t = i%4) are the low (t < 2) or high
        // nibbles of bytes 8(t%2)..8(t%2)+7
        const int ib = 2 * g + (i >> 2);
        const int ls = (int)(((hdr.y >> (4 * ib)) & 0xFu) | ((((hdr.x >> 16) >> (2 * ib)) & 3u) << 4)) - 32;
        const uint4 v = q[i >> 2];
        const int sh = 4 * ((i >> 1) & 1);
        const uint32_t w0 = (i & 1) ? v.z : v.x, w1 = (i & 1) ? v.w : v.y;
        return scale8(lut4((w0 >> sh) & 0x0F0F0F0Fu, tab), lut4((w1 >> sh) & 0x0F0F0F0Fu, tab), (_Float16)(float)ls, lo);
    }
};

template <>
struct BFrag<QKK_Q6_K> { // group g owns, of half g/2, l = 16(g%2)..16(g%2)+15 of all four quarters
    static constexpr int BYTES = Q6_K_BYTES, LAYOUT = 1;
    static constexpr bool SPLIT = true; // |q| <= 32 times |scale| <= 128
    uint4 qa, qb, qh; // ql[l], ql[l+32], qh[l]
    uint2 sc;         // the eight scales of the half
    uint16_t d;
    __device__ __forceinline__ void load(const uint8_t* row, uint32_t fi, int g)
    {
        const uint8_t* p = row + (size_t)fi * BYTES;
        const int n = g >> 1, gl = g & 1;
        qa = ldg<uint4>(p + 64 * n + 16 * gl);
        qb = ldg<uint4>(p + 64 * n + 32 + 16 * gl);
        qh = ldg<uint4>(p + Q6_K_QH + 32 * n + 16 * gl);
        sc = ldg<uint2>(p + Q6_K_SC + 8 * n);
        d = ldg<uint16_t>(p + Q6_K_D);
    }
    __device__ __forceinline__ float post() const { return h2f(d); }
    __device__ __forceinline__ half8 step(int i, int g, const MfmaTables&, half8& lo) const
    {
        const int m = i >> 1; // quarter: ql[l] low, ql[l+32] low, ql[l] high, ql[l+32] high nibbles
        const uint4 L = (m & 1) ? qb : qa;
        const uint32_t l0 = (i & 1) ? L.z : L.x, l1 = (i & 1) ? L.w : L.y;
        const uint32_t h0 = (i & 1) ? qh.z : qh.x, h1 = (i & 1) ? qh.w : qh.y;
        const uint32_t v0 = ((l0 >> (4 * (m >> 1))) & 0x0F0F0F0Fu) | (((h0 >> (2 * m)) & 0x03030303u) << 4);
        const uint32_t v1 = ((l1 >> (4 * (m >> 1))) & 0x0F0F0F0Fu) | (((h1 >> (2 * m)) & 0x03030303u) << 4);
        const uint32_t sw = m < 2 ? sc.x : sc.y; // scale 2m + g%2 of the half
        const int s = (int)(int8_t)((sw >> (16 * (m & 1) + 8 * (g & 1))) & 0xFFu);
        return scale8(bytes_to_half4(v0, 32.f), bytes_to_half4(v1, 32.f), (_Float16)(float)s, lo);
    }
};

// ---- cooperative streaming ----------------------------------------------------------------------------
// The weight rows of a sub-item are ONE contiguous byte range per tensor (consecutive rows of a
// row-major tensor), so the workgroup copies it to LDS in batches with fully coalesced 16-byte
// loads, double-buffered: the L1 sees every line once.  The eight waves split K: wave w owns
// fragment w % KS of every row (its slice of the 16 activation rows stays in registers as the
// MFMA A operand, hi + lo halves) and, when KS < 8, tile group w / KS.  Per batch every wave
// reads its fragments of the batch's tiles from LDS, runs the MFMAs, writes its partial
// 16x16 results to LDS; after a barrier the partials are summed in wave order (a fixed order:
// results are bit-reproducible) and handed to the epilogue.
constexpr int CW = 8;       // waves per workgroup
constexpr int CT = 64 * CW; // threads per workgroup

// ALT: the NS = 2 tensors take turns, batch 2q = tiles of tensor 0, batch 2q+1 = the same rows
// of tensor 1 (for blocks too large to double-buffer both tensors' tiles together).
// NA: tiles of 16 activation rows a wave keeps as A operands (every weight fragment is decoded once
// and applied to all of them).
// PB: partial-result buffers, 2 (one barrier per batch) or 1 (two barriers, less LDS).
template <int TYPE, int KS, int NS, int TG, bool ALT = false, int NA = 1, int PB = 2>
struct CoopGeom {
    static constexpr int G = CW / KS;                   // tile groups
    static constexpr int BT = G * TG;                   // row tiles per tensor and batch
    static constexpr int NSB = ALT ? 1 : NS;            // tensors per batch
    static constexpr uint32_t RB = (uint32_t)qkk_row_bytes_dev<TYPE>(256 * KS);
    static constexpr uint32_t TBYTES = 16 * RB;         // one tile of 16 rows: contiguous
    static constexpr uint32_t BBYTES = NSB * BT * TBYTES; // one batch in LDS
    static constexpr uint32_t PART_BYTES = NSB * BT * KS * NA * 64 * 16;
    static constexpr uint32_t LDS_BYTES = 2 * BBYTES + PB * PART_BYTES;
    static_assert(BBYTES % 16 == 0 && CW % KS == 0 && (!ALT || NS == 2), "geometry");
};

// The A operand of one wave: rows row_of(0..np-1) (rows >= np read as zero), K slice
// [k0, k0+256) in the cut of `LAYOUT` (see BFrag), split into hi + lo halves.
struct AFrag {
    half8 hi[8], lo[8];
};

template <int LAYOUT, typename RowOf>
__device__ __forceinline__ void load_afrag(AFrag& a, const float* __restrict__ X, uint32_t stride, uint32_t k0,
                                           uint32_t np, RowOf row_of, int lane, uint32_t first_row = 0)
{
    const uint32_t j = first_row + (lane & 15), g = lane >> 4;
    const float keep = j < np ? 1.f : 0.f;
    const float* src = X + (size_t)row_of(min(j, np - 1)) * stride + k0;
    float4 v[8][2];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t k = LAYOUT == 0 ? 64 * g + 8 * i : 128 * (g >> 1) + 32 * (i >> 1) + 16 * (g & 1) + 8 * (i & 1);
        v[i][0] = *(const float4*)(src + k);
        v[i][1] = *(const float4*)(src + k + 4);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float f[8] = {v[i][0].x, v[i][0].y, v[i][0].z, v[i][0].w, v[i][1].x, v[i][1].y, v[i][1].z, v[i][1].w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x = f[e] * keep;
            a.hi[i][e] = (_Float16)x;
            a.lo[i][e] = (_Float16)(x - (float)a.hi[i][e]);
        }
    }
}

// Streams n_batches batches of BT row tiles starting at base0 / base1 (tensor 0 / 1, first row
// of the sub-item) and calls epi(tile, lane, e, sum0, sum1, na) for every output: tile = row tile
// within the sub-item, lane%16 = row within the tile, 16*na + 4*(lane/16)+e = activation row,
// sum_s = tensor s's dot product.  One barrier per batch: batch b+1 is written to the other LDS buffer
// as soon as this wave is done with batch b (nobody reads that buffer any more), the partials
// alternate between two buffers as well, so fast waves run ahead into the next batch.
// CLAMP: `limit` is the offset from base0 of the tensor's last 16 bytes; loads beyond it re-read
// those (the caller ignores the rows that do not exist).
// STRIDED: the rows are longer than 256*KS weights and this call takes the RB bytes at base0 of
// each (a K range of every row): consecutive rows lie row_stride bytes apart, a row's piece is
// still contiguous and a multiple of 16 bytes, and LDS receives the pieces packed as before.
template <int TYPE, int KS, int NS, int TG, bool ALT, bool CLAMP, int NA = 1, int PB = 2, bool STRIDED = false,
          typename RowOf, typename Epi>
__device__ __forceinline__ void coop_stream(const uint8_t* __restrict__ base0, const uint8_t* __restrict__ base1,
                                            uint32_t n_batches, const float* __restrict__ A_src, uint32_t a_stride,
                                            uint32_t np, RowOf row_of, uint8_t* smem, const MfmaTables& tab, int tid,
                                            Epi epi, size_t limit = 0, uint32_t row_stride = 0)
{
    using Geo = CoopGeom<TYPE, KS, NS, TG, ALT, NA, PB>;
    constexpr int BT = Geo::BT, NSB = Geo::NSB, NTL = NSB * TG; // tiles per wave and batch
    constexpr uint32_t RB = Geo::RB, TBYTES = Geo::TBYTES, BBYTES = Geo::BBYTES, PBYTES = Geo::PART_BYTES;
    constexpr int PIECES = BBYTES / 16, PPT = BT * TBYTES / 16, NLD = (PIECES + CT - 1) / CT;
    constexpr uint32_t PPR = RB / 16; // STRIDED: pieces per row
    static_assert(!STRIDED || (RB % 16 == 0 && !ALT && NSB == 1), "strided rows: whole 16-byte pieces, one tensor");
    constexpr int OUTS = (NA * BT * 256 + CT - 1) / CT; // outputs per thread and batch
    const int lane = tid & 63, wave = tid >> 6, kw = wave % KS, tg = wave / KS, j = lane & 15, g = lane >> 4;
    const uint32_t steps = ALT ? 2 * n_batches : n_batches; // LDS batches

    // piece p of a batch: 16 bytes at offset (p % PPT)*16 of tensor p / PPT; LDS keeps the same order
    const uint8_t* src[NLD];
    size_t room[NLD]; // CLAMP: how far this piece may advance
#pragma unroll
    for (int n = 0; n < NLD; n++) {
        const uint32_t p = min((uint32_t)(tid + CT * n), (uint32_t)PIECES - 1);
        const uint32_t pp = p % PPT;
        size_t off = STRIDED ? (size_t)(pp / PPR) * row_stride + (size_t)(pp % PPR) * 16 : (size_t)pp * 16;
        if (CLAMP) { off = min(off, limit); room[n] = limit - off; }
        src[n] = ((NSB > 1 && p >= (uint32_t)PPT) ? base1 : base0) + off;
    }
    const size_t alt_delta = ALT ? (size_t)(base1 - base0) : 0;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 ld[NLD];
    const size_t batch_bytes = STRIDED ? (size_t)(BT * 16) * row_stride : (size_t)(BT * TBYTES);
    const auto adv_of = [&](uint32_t nx) -> size_t {
        nx = min(nx, steps - 1); // past the end: a harmless re-read
        return ALT ? (size_t)(nx >> 1) * batch_bytes + (nx & 1u) * alt_delta : (size_t)nx * batch_bytes;
    };
#pragma unroll
    for (int n = 0; n < NLD; n++) ld[n] = *(const u32x4*)src[n];
    AFrag a[NA]; // fetched and converted while the first batch is in flight
#pragma unroll
    for (int na = 0; na < NA; na++) load_afrag<BFrag<TYPE>::LAYOUT>(a[na], A_src, a_stride, 256 * kw, np, row_of, lane, 16 * na);
#pragma unroll
    for (int n = 0; n < NLD; n++)
        if (PIECES % CT == 0 || n + 1 < NLD || tid + CT * n < PIECES) *(u32x4*)(smem + (size_t)(tid + CT * n) * 16) = ld[n];
    __syncthreads();
    float saved[OUTS]; // ALT: tensor 0's sums wait here for tensor 1's
#pragma unroll
    for (int o = 0; o < OUTS; o++) saved[o] = 0.f;

#pragma unroll 1
    for (uint32_t b = 0; b < steps; b++) {
        const uint32_t buf = b & 1u;
        {   // next batch: lands during the MFMA phase
            const size_t adv = adv_of(b + 1);
#pragma unroll
            for (int n = 0; n < NLD; n++) // a signed step: with two tensors the way from one to the other may lead down
                ld[n] = *(const u32x4*)(src[n] + (ptrdiff_t)(CLAMP ? min(adv, room[n]) : adv));
        }
        // this wave's fragments of the batch: tiles tg*TG .. +TG of every tensor in it
        BFrag<TYPE> f[NTL];
#pragma unroll
        for (int s = 0; s < NSB; s++)
#pragma unroll
            for (int t = 0; t < TG; t++)
                f[s * TG + t].load(smem + buf * BBYTES + ((size_t)(s * BT + tg * TG + t) * 16 + j) * RB, kw, g);
        float4v acc[NTL][NA];
#pragma unroll
        for (int t = 0; t < NTL; t++)
#pragma unroll
            for (int na = 0; na < NA; na++) acc[t][na] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int t = 0; t < NTL; t++) {
                half8 bl;
                const half8 bh = f[t].step(i, g, tab, bl);
#pragma unroll
                for (int na = 0; na < NA; na++) {
                    acc[t][na] = mfma16x32(a[na].hi[i], bh, acc[t][na]);
                    acc[t][na] = mfma16x32(a[na].lo[i], bh, acc[t][na]);
                    if constexpr (BFrag<TYPE>::SPLIT) acc[t][na] = mfma16x32(a[na].hi[i], bl, acc[t][na]);
                }
            }
            __builtin_amdgcn_sched_barrier(0); // keep the decode of later steps from piling up in registers
        }
        float* part = (float*)(smem + 2 * BBYTES + (PB > 1 ? buf : 0u) * PBYTES); // [NA][NSB*BT][KS][64 lanes][4]
#pragma unroll
        for (int s = 0; s < NSB; s++)
#pragma unroll
            for (int t = 0; t < TG; t++) {
                const float sc = f[s * TG + t].post();
#pragma unroll
                for (int na = 0; na < NA; na++) {
                    const float4v r = acc[s * TG + t][na];
                    *(float4*)(part + ((((size_t)na * NSB * BT + s * BT + tg * TG + t) * KS + kw) * 64 + lane) * 4) =
                        float4{sc * r[0], sc * r[1], sc * r[2], sc * r[3]};
                }
            }
#pragma unroll
        for (int n = 0; n < NLD; n++)
            if (PIECES % CT == 0 || n + 1 < NLD || tid + CT * n < PIECES)
                *(u32x4*)(smem + (buf ^ 1u) * BBYTES + (size_t)(tid + CT * n) * 16) = ld[n];
        __syncthreads(); // partials of batch b complete, batch b+1 in place
#pragma unroll
        for (int oo = 0; oo < OUTS; oo++) {
            const uint32_t o = tid + CT * oo;
            if (NA * BT * 256 % CT != 0 && o >= (uint32_t)NA * BT * 256) break;
            const uint32_t na = o / (BT * 256), bt = (o >> 8) % BT, e = (o >> 6) & 3u, ln = o & 63u;
            const float* pa = part + (size_t)na * (NSB * BT * KS * 256);
            float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
            for (int w = 0; w < KS; w++) {
                sum0 += pa[(((size_t)bt * KS + w) * 64 + ln) * 4 + e];
                if (NSB > 1) sum1 += pa[(((size_t)(BT + bt) * KS + w) * 64 + ln) * 4 + e];
            }
            if (!ALT) epi(b * BT + bt, ln, e, sum0, sum1, na);
            else if (b & 1u) epi((b >> 1) * BT + bt, ln, e, saved[oo], sum0, na);
            else saved[oo] = sum0;
        }
        if (PB == 1) __syncthreads(); // the single partial buffer is free again
    }
    __syncthreads(); // the buffers are free for the next call
}

} // namespace qk
