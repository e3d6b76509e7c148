// qk_moe_mfma.hip -- expert-major gate/up and down projections on MFMA for several tokens
// (decode slots or a prefill chunk).
//
// A work item is one expert with the (token, pick) pairs routed to it, or the shared expert
// with 16 consecutive tokens, cut into sub-items by weight-row tiles.  A workgroup of 8 waves
// takes a sub-item: it gathers 16 of the item's activation rows into LDS as half hi + half lo
// planes in MFMA fragment order, then every wave streams its weight rows ONCE from HBM and
// applies them to all 16 rows with v_mfma_f32_16x16x32_f16; the activation fragments a wave
// reads from LDS are shared by all the weight tiles it holds.  Orientation, exactness and
// post-scaling: see qk_mfma.h -- the weight operand carries the block's integers, block scales
// are applied to the MFMA result in fp32.
// (reference shaders/moe_gateup_iq3_grouped_coopmat.comp:46-217, moe_down_iq4_grouped_coopmat.comp:45-166,
//  moe_gateup_q8_coopmat.comp, moe_down_q8_coopmat.comp.)
#include "qk_mfma.h"
#include "qk_moe_common.h"

#include <algorithm>

namespace qk {

struct MfmaTables {
    uint32_t grid[256]; // IQ3_XXS codewords, four magnitudes per dword
    uint32_t iq4[4];    // IQ4 codebook, sixteen int8 in four dwords
};

__device__ static void fill_mfma_tables(MfmaTables& t, int tid, int nthreads)
{
    for (int i = tid; i < 256; i += nthreads) t.grid[i] = g_iq3xxs_grid[i];
    if (tid < 4) {
        constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (i / 4 == tid) w |= (uint32_t)(uint8_t)kv[i] << (8 * (i % 4));
        t.iq4[tid] = w;
    }
}

// ---- a lane's share of one 256-weight fragment of row (l%16), in the B-operand cut -----------------
// What limits these kernels is the number of L1 accesses, one per lane and load instruction,
// so lane group g = l/16 owns 64 of the fragment's 256 weights chosen so that its bytes are
// CONTIGUOUS in the block (LAYOUT, see stage_rows256) and fetches them with two or three wide
// loads.  Step i of 8 feeds eight of them to one K = 32 MFMA.  The four lane groups of a step
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
    // four magnitudes (bytes of cw, each <= 62) with sign bits s4 -> four halves +-mag, exact:
    // the byte 0x80 +- mag under the exponent byte 0x64 is the half 1152 +- mag
    __device__ __forceinline__ static half4 signed4(uint32_t cw, uint32_t s4)
    {
        const uint32_t t = ((s4 & 15u) * 0x00204081u) & 0x01010101u;
        const uint32_t m = (t << 8) - t;                               // 0xFF in the bytes to negate
        const uint32_t pos = cw + 0x80808080u, neg = 0x80808080u - cw; // no carry between bytes
        return bytes_to_half4((neg & m) | (pos & ~m), 128.f);
    }
    __device__ __forceinline__ half8 step(int i, int, const MfmaTables& tab, half8&) const
    {
        const uint32_t a = (i >> 2) ? aux.y : aux.x;
        const uint32_t s7 = (a >> (7 * (i & 3))) & 127u;
        const uint32_t s8 = s7 | ((__builtin_popcount(s7) & 1u) << 7);
        const uint32_t w = (i >> 1) == 0 ? idx.x : (i >> 1) == 1 ? idx.y : (i >> 1) == 2 ? idx.z : idx.w;
        const uint32_t pr = w >> (16 * (i & 1));
        const half4 lo = signed4(tab.grid[pr & 255u], s8), hi = signed4(tab.grid[(pr >> 8) & 255u], s8 >> 4);
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

// Fragment number `fi` of the staged tile for NT weight tiles at once: the activation
// fragments are read from LDS once per step and reused by all NT tiles; the eight steps chain
// through the MFMA accumulator and the row's factor is applied once.
template <int TYPE, int NT>
__device__ __forceinline__ void mac_multi(const BFrag<TYPE>* f, const _Float16* __restrict__ s_hi,
                                          const _Float16* __restrict__ s_lo, uint32_t fi, int lane, int g,
                                          const MfmaTables& tab, float4v* acc)
{
    float4v part[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) part[t] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const size_t off = ((size_t)(fi * 8 + i) * 64 + lane) * 8;
        const half8 ah = *(const half8*)(s_hi + off), al = *(const half8*)(s_lo + off);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            half8 bl;
            const half8 b = f[t].step(i, g, tab, bl);
            part[t] = mfma16x32(ah, b, part[t]);
            part[t] = mfma16x32(al, b, part[t]);
            if constexpr (BFrag<TYPE>::SPLIT) part[t] = mfma16x32(ah, bl, part[t]);
        }
        __builtin_amdgcn_sched_barrier(0); // keep the decode of later steps from piling up in registers
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const float sc = f[t].post();
#pragma unroll
        for (int e = 0; e < 4; e++) acc[t][e] += sc * part[t][e];
    }
}

// Streams NT weight rows per lane (rowp[t] = this lane's row of tile t, at the first staged
// weight) over `nfrag` fragments of the staged activation tile through a ring of DEPTH
// fragment sets.  prime() issues the first DEPTH loads and needs nothing from LDS, so it is
// called BEFORE the activation rows are staged: HBM latency overlaps the staging.  In run()
// the loads of fragment b+DEPTH are issued as soon as fragment b has been consumed; loads
// past the end re-read the last fragment (no branch around a load).
template <int TYPE, int NT, int DEPTH>
struct Stream {
    using F = BFrag<TYPE>;
    F f[DEPTH][NT];
    __device__ __forceinline__ void prime(const uint8_t* const* rowp, uint32_t nfrag, int g)
    {
#pragma unroll
        for (int dd = 0; dd < DEPTH; dd++)
#pragma unroll
            for (int t = 0; t < NT; t++) f[dd][t].load(rowp[t], min((uint32_t)dd, nfrag - 1), g);
    }
    __device__ __forceinline__ void run(const uint8_t* const* rowp, uint32_t nfrag, const _Float16* s_hi,
                                        const _Float16* s_lo, int lane, int g, const MfmaTables& tab, float4v* acc)
    {
#pragma unroll 1
        for (uint32_t b = 0; b < nfrag; b += DEPTH) {
#pragma unroll
            for (int dd = 0; dd < DEPTH; dd++) {
                if (DEPTH == 1 || b + dd < nfrag) mac_multi<TYPE, NT>(f[dd], s_hi, s_lo, b + dd, lane, g, tab, acc);
#pragma unroll
                for (int t = 0; t < NT; t++)
                    f[dd][t].load(rowp[t], min(b + dd + DEPTH, nfrag - 1), g);
            }
        }
    }
};

constexpr int GU_WAVES = 8; // waves per gate/up workgroup
constexpr int GU_TPW = 2;   // row tiles per wave: its gate and up tile share every activation fragment
constexpr int DN_WAVES = 8;
constexpr int DN_TPW = 4;   // row tiles per wave in the down launch

// Work items: first the shared expert's tiles of 16 consecutive tokens (they cannot be split
// by pairs, so they start first), then the routed experts with their pair lists.  Every item
// is cut into sub-items that take different weight-row tiles, so one expert's rows are
// streamed by several workgroups (each stages the item's activation rows itself).
struct Item {
    bool shared;
    uint32_t expert, first, count; // routed: pairs [first, first+count) of ws.pairs; shared: tokens
    uint32_t sub;
};

__device__ __forceinline__ uint32_t item_count(uint32_t n_active, uint32_t N, uint32_t subs_shared, uint32_t subs)
{
    return (N + 15) / 16 * subs_shared + n_active * subs;
}

__device__ __forceinline__ Item get_item(const MoeWs& ws, uint32_t index, uint32_t subs_shared, uint32_t subs, uint32_t N)
{
    Item it;
    const uint32_t n_sh = (N + 15) / 16 * subs_shared;
    if (index < n_sh) {
        it.sub = index % subs_shared;
        it.shared = true; it.expert = 0; it.first = index / subs_shared * 16u; it.count = min(16u, N - it.first);
    } else {
        const uint32_t w = (index - n_sh) / subs;
        it.sub = (index - n_sh) % subs;
        const ActiveExpert a = ws.active[w];
        it.shared = false; it.expert = a.expert; it.first = a.first; it.count = a.count;
    }
    return it;
}

// ---- gate/up + SiLU --------------------------------------------------------------------------------
// One sub-item: GU_WAVES*GU_TPW row tiles of gate and up for up to 16 staged rows.  H = 2048*NCHUNK.
// TYPE = format of the gate/up tensors of this item (IQ3_XXS experts, Q8_0 shared expert).
// TPW = row tiles per wave (their gate and up rows share every activation fragment).
template <int TYPE, int NCHUNK, int TPW, int DEPTH>
__device__ __forceinline__ void gateup_tile(const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up,
                                            size_t row_bytes, const float* __restrict__ X, float* __restrict__ h,
                                            const MoeDims& d, uint32_t tile0, uint32_t np, _Float16* s_hi,
                                            _Float16* s_lo, const uint32_t* s_tok, const uint32_t* s_slot,
                                            const MfmaTables& tab, int tid)
{
    constexpr int NT = 2 * TPW; // weight tiles per lane: gate q0, up q0, gate q1, up q1 ...
    constexpr uint32_t NFRAG = 2048 / 256; // fragments per staged chunk
    const int lane = tid & 63, j = lane & 15, g = lane >> 4;
    const uint8_t* rowp[NT];
#pragma unroll
    for (int q = 0; q < TPW; q++) {
        const size_t ro = (size_t)((tile0 + GU_WAVES * q) * 16 + j) * row_bytes;
        rowp[2 * q] = gate + ro;
        rowp[2 * q + 1] = up + ro;
    }
    float4v acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int ch = 0; ch < NCHUNK; ch++) {
        Stream<TYPE, NT, DEPTH> st;
        if (ch) {
            __syncthreads(); // the previous chunk's fragments are consumed
#pragma unroll
            for (int t = 0; t < NT; t++) rowp[t] += qkk_row_bytes_dev<TYPE>(2048);
        }
        st.prime(rowp, NFRAG, g); // in flight while the activation rows are staged
        stage_rows256<BFrag<TYPE>::LAYOUT, 2048, 64 * GU_WAVES>(s_hi, s_lo, X + ch * 2048, d.H, np,
                                                               [&](uint32_t r) { return s_tok[r]; }, tid);
        __syncthreads();
        st.run(rowp, NFRAG, s_hi, s_lo, lane, g, tab, acc);
    }
    // lane holds rows (tile0 + GU_WAVES*q)*16 + j for staged rows 4g+e
#pragma unroll
    for (int q = 0; q < TPW; q++) {
        const uint32_t row = (tile0 + GU_WAVES * q) * 16 + j;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t r = 4 * g + e;
            if (r < np) {
                const float gg = acc[2 * q][e], uu = acc[2 * q + 1][e];
                h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * d.F + row] = (gg / (1.f + expf(-gg))) * uu;
            }
        }
    }
}

template <int NCHUNK>
__global__ __launch_bounds__(64 * GU_WAVES) void moe_gateup_mfma_kernel(const uint8_t* __restrict__ gate_exps,
                                                                        const uint8_t* __restrict__ up_exps,
                                                                        const uint8_t* __restrict__ gate_shexp,
                                                                        const uint8_t* __restrict__ up_shexp,
                                                                        const float* __restrict__ X, MoeWs ws,
                                                                        MoeDims d, uint32_t N)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    _Float16* s_hi = (_Float16*)smem;
    _Float16* s_lo = s_hi + 16 * 2048;
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    const int tid = threadIdx.x, wave = tid >> 6;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, 64 * GU_WAVES);
    const uint32_t n_active = *ws.n_active;
    const uint32_t subs_sh = F / (16 * GU_WAVES), subs = F / (16 * GU_WAVES * GU_TPW);
    const uint32_t n_items = item_count(n_active, N, subs_sh, subs);

    for (uint32_t w = blockIdx.x; w < n_items; w += gridDim.x) {
        const Item it = get_item(ws, w, subs_sh, subs, N);
        const uint32_t tile0 = it.sub * GU_WAVES * (it.shared ? 1 : GU_TPW) + wave; // this wave: tile0 + GU_WAVES*q
        for (uint32_t t0 = 0; t0 < it.count; t0 += 16) {
            const uint32_t np = it.shared ? it.count : min(16u, it.count - t0);
            __syncthreads(); // previous tile fully consumed
            if (tid < 16) {
                uint32_t tok = 0, slot = 0;
                if ((uint32_t)tid < np) {
                    if (it.shared) { tok = it.first + tid; slot = d.k; }
                    else { const uint32_t pr = ws.pairs[it.first + t0 + tid]; tok = pr >> 4; slot = pr & 15u; }
                }
                s_tok[tid] = tok;
                s_slot[tid] = slot;
            }
            __syncthreads();
            if (it.shared) {
                gateup_tile<QKK_Q8_0, NCHUNK, 1, 3>(gate_shexp, up_shexp, (size_t)H / 32 * Q8_0_BYTES, X, ws.h, d, tile0, np,
                                                 s_hi, s_lo, s_tok, s_slot, tab, tid);
                break;
            }
            const size_t rb = (size_t)H / 256 * IQ3_XXS_BYTES, eo = (size_t)it.expert * F * rb;
            gateup_tile<QKK_IQ3_XXS, NCHUNK, GU_TPW, 3>(gate_exps + eo, up_exps + eo, rb, X, ws.h, d, tile0, np, s_hi, s_lo,
                                                s_tok, s_slot, tab, tid);
        }
    }
}

// ---- down: per-pair contributions -----------------------------------------------------------------
// contrib[(token*(k+1) + slot)*H + o] = weight * (D[o] . h[token][slot]); slot k = shared expert.
// A sub-item is DN_WAVES*DN_TPW row tiles of 16.  FB = F/256.
template <int TYPE, int FB, int NT, int DEPTH>
__device__ __forceinline__ void down_tile(const uint8_t* __restrict__ W, const float* __restrict__ h,
                                          float* __restrict__ contrib, const MoeDims& d, uint32_t tile0, uint32_t np,
                                          _Float16* s_hi, _Float16* s_lo, const uint32_t* s_tok, const uint32_t* s_slot,
                                          const float* s_wt, const MfmaTables& tab, int tid)
{
    constexpr uint32_t NFRAG = FB;
    const size_t RB = qkk_row_bytes_dev<TYPE>(256 * FB);
    const int lane = tid & 63, j = lane & 15, g = lane >> 4;
    const auto row_of = [&](uint32_t r) { return s_tok[r] * (d.k + 1) + s_slot[r]; };
#pragma unroll 1
    for (int q0 = 0; q0 < DN_TPW; q0 += NT) {
        const uint8_t* rowp[NT];
#pragma unroll
        for (int q = 0; q < NT; q++) rowp[q] = W + (size_t)((tile0 + DN_WAVES * (q0 + q)) * 16 + j) * RB;
        Stream<TYPE, NT, DEPTH> st;
        st.prime(rowp, NFRAG, g);
        if (q0 == 0) {
            stage_rows256<BFrag<TYPE>::LAYOUT, 256 * FB, 64 * DN_WAVES>(s_hi, s_lo, h, d.F, np, row_of, tid);
            __syncthreads();
        }
        float4v acc[NT];
#pragma unroll
        for (int q = 0; q < NT; q++) acc[q] = float4v{0.f, 0.f, 0.f, 0.f};
        st.run(rowp, NFRAG, s_hi, s_lo, lane, g, tab, acc);
#pragma unroll
        for (int q = 0; q < NT; q++) {
            const uint32_t row = (tile0 + DN_WAVES * (q0 + q)) * 16 + j;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t r = 4 * g + e;
                if (r < np) contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * d.H + row] = s_wt[r] * acc[q][e];
            }
        }
    }
}

template <int TYPE_DN, int FB>
__global__ __launch_bounds__(64 * DN_WAVES) void moe_down_mfma_kernel(const uint8_t* __restrict__ down_exps,
                                                                      const uint8_t* __restrict__ down_shexp,
                                                                      MoeWs ws, const qkk_sel* __restrict__ sel,
                                                                      MoeDims d, uint32_t N)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    _Float16* s_hi = (_Float16*)smem;
    _Float16* s_lo = s_hi + 16 * 256 * FB;
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x, wave = tid >> 6;
    const uint32_t H = d.H;
    fill_mfma_tables(tab, tid, 64 * DN_WAVES);
    const uint32_t n_active = *ws.n_active;
    const uint32_t subs = H / (16 * DN_WAVES * DN_TPW);
    const uint32_t n_items = item_count(n_active, N, subs, subs);

    for (uint32_t w = blockIdx.x; w < n_items; w += gridDim.x) {
        const Item it = get_item(ws, w, subs, subs, N);
        const uint32_t tile0 = it.sub * DN_WAVES * DN_TPW + wave; // this wave: tile0 + DN_WAVES*q
        for (uint32_t t0 = 0; t0 < it.count; t0 += 16) {
            const uint32_t np = it.shared ? it.count : min(16u, it.count - t0);
            __syncthreads();
            if (tid < 16) {
                uint32_t tok = 0, slot = 0;
                float wt = 0.f;
                if ((uint32_t)tid < np) {
                    if (it.shared) { tok = it.first + tid; slot = d.k; wt = sel[tok].w_shared; }
                    else {
                        const uint32_t pr = ws.pairs[it.first + t0 + tid];
                        tok = pr >> 4; slot = pr & 15u; wt = sel[tok].w[slot];
                    }
                }
                s_tok[tid] = tok; s_slot[tid] = slot; s_wt[tid] = wt;
            }
            __syncthreads();
            if (it.shared) {
                down_tile<QKK_Q8_0, FB, 2, (FB < 2 ? 1 : 2)>(down_shexp, ws.h, ws.contrib, d, tile0, np, s_hi, s_lo, s_tok,
                                                            s_slot, s_wt, tab, tid);
                break;
            }
            const size_t RB = qkk_row_bytes_dev<TYPE_DN>(256 * FB);
            down_tile<TYPE_DN, FB, 2, (FB < 2 ? 1 : 2)>(down_exps + (size_t)it.expert * H * RB, ws.h, ws.contrib, d,
                                                            tile0, np, s_hi, s_lo, s_tok, s_slot, s_wt, tab, tid);
        }
    }
}

// ---- fold: Y[t][o] = sum over the k+1 slots, in slot order --------------------------------------------
__global__ __launch_bounds__(256) void moe_fold_kernel(MoeWs ws, float* __restrict__ Y, MoeDims d, uint32_t N)
{
    const uint32_t quads = d.H / 4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)N * quads; i += (size_t)gridDim.x * 256) {
        const uint32_t t = (uint32_t)(i / quads), o = (uint32_t)(i % quads) * 4;
        float4 s = float4{0.f, 0.f, 0.f, 0.f};
        for (uint32_t sl = 0; sl <= d.k; sl++) {
            const float4 c = *(const float4*)(ws.contrib + ((size_t)t * (d.k + 1) + sl) * d.H + o);
            s.x += c.x; s.y += c.y; s.z += c.z; s.w += c.w;
        }
        *(float4*)(Y + (size_t)t * d.H + o) = s;
    }
}

// ---- host -----------------------------------------------------------------------------------------------
static void set_lds_attr(const void* fn)
{
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
}

static void launch_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, const MoeDims& d, uint32_t N,
                          uint32_t blocks, hipStream_t st)
{
    const size_t lds = (size_t)2 * 16 * 2048 * sizeof(_Float16);
    const uint8_t *ge = (const uint8_t*)L->gate_exps, *ue = (const uint8_t*)L->up_exps,
                  *gs = (const uint8_t*)L->gate_shexp, *us = (const uint8_t*)L->up_shexp;
    if (d.H == 2048) {
        static bool once = (set_lds_attr((const void*)moe_gateup_mfma_kernel<1>), true);
        (void)once;
        hipLaunchKernelGGL(moe_gateup_mfma_kernel<1>, dim3(blocks), dim3(64 * GU_WAVES), lds, st, ge, ue, gs, us, X, ws, d, N);
    } else {
        static bool once = (set_lds_attr((const void*)moe_gateup_mfma_kernel<2>), true);
        (void)once;
        hipLaunchKernelGGL(moe_gateup_mfma_kernel<2>, dim3(blocks), dim3(64 * GU_WAVES), lds, st, ge, ue, gs, us, X, ws, d, N);
    }
}

template <int TYPE, int FB>
static void launch_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d, uint32_t N,
                        uint32_t blocks, hipStream_t st)
{
    const size_t lds = (size_t)2 * 16 * 256 * FB * sizeof(_Float16);
    static bool once = (set_lds_attr((const void*)moe_down_mfma_kernel<TYPE, FB>), true);
    (void)once;
    hipLaunchKernelGGL((moe_down_mfma_kernel<TYPE, FB>), dim3(blocks), dim3(64 * DN_WAVES), lds, st,
                       (const uint8_t*)L->down_exps, (const uint8_t*)L->down_shexp, ws, sel, d, N);
}

// Gate/up, down and fold for N >= 2 rows; the router record and the pair lists are in place.
void moe_mfma_launch(const qkk_moe_layer* L, const float* X, float* Y, const qkk_sel* sel, const MoeWs& ws,
                     const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st)
{
    const uint32_t max_items = (uint32_t)std::min<uint64_t>(d.E, (uint64_t)N * d.k) + (N + 15) / 16;
    // down: 8-wave workgroups, several share a CU (the staged tile is 16*F*4 bytes)
    const uint32_t blocks = std::min(max_items * (d.H / (16 * DN_WAVES * DN_TPW)), persistent_blocks() / 2);
    if (stages & QKK_STAGE_GATEUP) {
        const uint32_t gu_items = (uint32_t)std::min<uint64_t>(d.E, (uint64_t)N * d.k) * (d.F / (16 * GU_WAVES * GU_TPW)) +
                                  (N + 15) / 16 * (d.F / (16 * GU_WAVES));
        const uint32_t gu_blocks = std::min(gu_items, persistent_blocks() / 4);
        launch_gateup(L, X, ws, d, N, gu_blocks, st);
    }
    if (stages & QKK_STAGE_DOWN) {
        if (L->down_type == QKK_IQ4_XS) {
            if (d.F == 256) launch_down<QKK_IQ4_XS, 1>(L, ws, sel, d, N, blocks, st);
            else if (d.F == 512) launch_down<QKK_IQ4_XS, 2>(L, ws, sel, d, N, blocks, st);
            else launch_down<QKK_IQ4_XS, 4>(L, ws, sel, d, N, blocks, st);
        } else {
            if (d.F == 256) launch_down<QKK_Q6_K, 1>(L, ws, sel, d, N, blocks, st);
            else if (d.F == 512) launch_down<QKK_Q6_K, 2>(L, ws, sel, d, N, blocks, st);
            else launch_down<QKK_Q6_K, 4>(L, ws, sel, d, N, blocks, st);
        }
        const uint32_t fb = (uint32_t)std::min<uint64_t>(((uint64_t)N * d.H / 4 + 255) / 256, persistent_blocks());
        hipLaunchKernelGGL(moe_fold_kernel, dim3(fb), dim3(256), 0, st, ws, Y, d, N);
    }
}

} // namespace qk
