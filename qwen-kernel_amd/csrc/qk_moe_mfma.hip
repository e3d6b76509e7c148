// qk_moe_mfma.hip -- expert-major gate/up and down projections on MFMA for several tokens
// (decode slots or a prefill chunk).
//
// A work item is one expert with the (token, pick) pairs routed to it, or the shared expert
// with 16 consecutive tokens, cut into sub-items by weight rows.  A workgroup of 8 waves takes
// a sub-item: its weight rows are one contiguous byte range, which the workgroup copies to LDS
// in double-buffered batches with coalesced 16-byte loads; the waves split K (each keeps its
// 256-wide slice of the 16 activation rows in registers as hi + lo half operands), decode
// their fragments from LDS into v_mfma_f32_16x16x32_f16 weight operands, and their partial
// 16x16 results are summed through LDS in a fixed order.  Each weight byte is read from HBM
// once per 16 rows; the L1 sees each line once.  Orientation and exactness: see qk_mfma.h.
// (reference shaders/moe_gateup_iq3_grouped_coopmat.comp:46-217, moe_down_iq4_grouped_coopmat.comp:45-166,
//  moe_gateup_q8_coopmat.comp, moe_down_q8_coopmat.comp.)
#include "qk_coop.h"
#include "qk_moe_common.h"

#include <algorithm>

namespace qk {

// How a launch's batches are divided: workgroup g of G takes the batches that start inside its equal
// share of the total cost (shared-expert batches first, cost cs each, then routed ones, cost cr each):
// the same work for every workgroup to within one batch, whatever the number of active experts.
struct Share {
    uint32_t s0, s1, r0, r1; // shared batches [s0, s1), routed batches [r0, r1)
};

__device__ __forceinline__ Share my_share(uint32_t g, uint32_t G, uint32_t ns, uint32_t cs, uint32_t nr, uint32_t cr)
{
    const uint64_t US = (uint64_t)ns * cs, U = US + (uint64_t)nr * cr;
    const uint64_t u0 = U * g / G, u1 = U * (g + 1) / G;
    const auto cdiv = [](uint64_t a, uint32_t b) { return (uint32_t)((a + b - 1) / b); };
    Share sh;
    sh.s0 = min(cdiv(min(u0, US), cs), ns);
    sh.s1 = min(cdiv(min(u1, US), cs), ns);
    sh.r0 = u0 > US ? min(cdiv(u0 - US, cr), nr) : 0u;
    sh.r1 = u1 > US ? min(cdiv(u1 - US, cr), nr) : 0u;
    return sh;
}

// Work items.  The shared expert is one dense expert for every token: its items are tiles of 16
// consecutive tokens; it depends on nothing the router produces, so its launches run on a side
// stream next to the router and the routed experts.  A routed item is one active expert with its
// pair list.  A workgroup's share of the batches falls into runs, each inside one item: the
// workgroup loads the item's activation rows and streams the run's weight rows.
struct Item {
    uint32_t expert, first, count; // routed: pairs [first, first+count) of ws.pairs; shared: tokens
};

// item w of the launch (w < number of token tiles, or < active_count())
template <bool SHARED>
__device__ __forceinline__ Item get_item(const MoeWs& ws, uint32_t w, const MoeDims& d, uint32_t N)
{
    Item it;
    if (SHARED) {
        it.expert = 0; it.first = w * 16u; it.count = min(16u, N - it.first);
    } else {
        const ActiveExpert a = active_expert(ws, w, d, N);
        it.expert = a.expert; it.first = a.first; it.count = a.count;
    }
    return it;
}

// this workgroup's batches [b0, b1) of the launch's n_items * tot
template <bool SHARED>
__device__ __forceinline__ void my_batches(const MoeWs& ws, const MoeDims& d, uint32_t N, uint32_t tot, uint32_t& b0,
                                           uint32_t& b1)
{
    const uint32_t n_items = SHARED ? (N + 15) / 16 : active_count(ws, d);
    // Where whole sub-items of a power-of-two length fill at least nine tenths of the grid, they are
    // taken as they are (a run never crosses an item, so no workgroup loads two activation tiles);
    // otherwise equal shares.
    for (uint32_t nb = tot; nb >= 1; nb >>= 1) {
        const uint64_t subs = (uint64_t)n_items * (tot / nb);
        if (subs > gridDim.x) break;
        if (subs * 10 >= (uint64_t)gridDim.x * 9 && tot % nb == 0) {
            b0 = blockIdx.x < subs ? blockIdx.x * nb : 0u;
            b1 = blockIdx.x < subs ? b0 + nb : 0u;
            return;
        }
    }
    const Share sh = my_share(blockIdx.x, gridDim.x, 0, 1, n_items * tot, 1);
    b0 = sh.r0;
    b1 = sh.r1;
}

// rows of the staged tile: s_tok[r] = token, s_slot[r] = h / contrib slot (k = shared expert)
template <bool SHARED>
__device__ __forceinline__ void stage_pairs(const MoeWs& ws, const Item& it, uint32_t t0, uint32_t np,
                                            const MoeDims& d, uint32_t N, uint32_t* s_tok, uint32_t* s_slot, int tid)
{
    if (tid < 16) {
        uint32_t tok = 0, slot = 0;
        if ((uint32_t)tid < np) {
            if (SHARED) { tok = it.first + tid; slot = d.k; }
            else pair_at(ws, it.first + t0 + tid, d, N, tok, slot);
        }
        s_tok[tid] = tok;
        s_slot[tid] = slot;
    }
}

// ---- gate/up + SiLU --------------------------------------------------------------------------------
// n_embd = 2048: the eight waves take one 256-weight fragment each.  A batch is one row tile; the
// gate tile and the up tile of the same rows take turns (ALT), which keeps the routed kernel at
// 121 VGPRs and 41 KB of LDS: two workgroups per CU.
template <bool SHARED>
using GuGeo = CoopGeom<SHARED ? QKK_Q8_0 : QKK_IQ3_XXS, 8, 2, 1, true>;

template <bool SHARED>
__global__ __launch_bounds__(CT, SHARED ? 2 : 4) void moe_gateup_mfma_kernel(const uint8_t* __restrict__ gate,
                                                                             const uint8_t* __restrict__ up,
                                                                             const float* __restrict__ X, MoeWs ws,
                                                                             MoeDims d, uint32_t N)
{
    using Geo = GuGeo<SHARED>;
    constexpr int TYPE = SHARED ? QKK_Q8_0 : QKK_IQ3_XXS;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t tot = F / (16 * Geo::BT); // batches per item
    uint32_t b0, b1;
    my_batches<SHARED>(ws, d, N, tot, b0, b1);

    for (uint32_t b = b0; b < b1;) {
        const uint32_t w = b / tot, f0 = b % tot, nbat = min(tot - f0, b1 - b);
        const Item it = get_item<SHARED>(ws, w, d, N);
        const uint32_t row0 = f0 * Geo::BT * 16;
        const size_t off = ((size_t)it.expert * F + row0) * Geo::RB;
        for (uint32_t t0 = 0; t0 < it.count; t0 += 16) {
            const uint32_t np = min(16u, it.count - t0);
            __syncthreads(); // previous tile fully consumed
            stage_pairs<SHARED>(ws, it, t0, np, d, N, s_tok, s_slot, tid);
            __syncthreads();
            coop_stream<TYPE, 8, 2, 1, true, false>(gate + off, up + off, nbat, X, H, np, [&](uint32_t r) { return s_tok[r]; },
                smem, tab, tid, [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * F + row0 + tile * 16 + (ln & 15u)] =
                            (sum0 / (1.f + expf(-sum0))) * sum1;
                });
        }
        b += nbat;
    }
}

// ---- down: per-pair contributions -----------------------------------------------------------------
// contrib[(token*(k+1) + slot)*H + o] = weight * (D[o] . h[token][slot]) for the routed slots; slot k
// (shared expert) holds the unweighted product, its sigmoid gate is applied by the fold (so the
// shared expert does not wait for the router).  K = F = 256*FB: FB waves split K, 8/FB tile groups
// split the batch's tiles.
template <int TYPE, int FB>
using DnGeo = CoopGeom<TYPE, FB, 1, (TYPE == QKK_IQ4_XS ? 2 : 1)>;

template <int TYPE, int FB, bool SHARED>
__global__ __launch_bounds__(CT) void moe_down_mfma_kernel(const uint8_t* __restrict__ down, MoeWs ws,
                                                           const qkk_sel* __restrict__ sel, MoeDims d, uint32_t N)
{
    using Geo = DnGeo<TYPE, FB>;
    constexpr int TG = TYPE == QKK_IQ4_XS ? 2 : 1;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t tot = H / (16 * Geo::BT);
    uint32_t b0, b1;
    my_batches<SHARED>(ws, d, N, tot, b0, b1);

    for (uint32_t b = b0; b < b1;) {
        const uint32_t w = b / tot, f0 = b % tot, nbat = min(tot - f0, b1 - b);
        const Item it = get_item<SHARED>(ws, w, d, N);
        const uint32_t row0 = f0 * Geo::BT * 16;
        const uint8_t* base = down + ((size_t)it.expert * H + row0) * Geo::RB;
        for (uint32_t t0 = 0; t0 < it.count; t0 += 16) {
            const uint32_t np = min(16u, it.count - t0);
            __syncthreads();
            stage_pairs<SHARED>(ws, it, t0, np, d, N, s_tok, s_slot, tid);
            __syncthreads();
            if (tid < 16) s_wt[tid] = (SHARED || (uint32_t)tid >= np) ? 1.f : sel[s_tok[tid]].w[s_slot[tid]];
            __syncthreads();
            coop_stream<TYPE, FB, 1, TG, false, false>(base, nullptr, nbat, ws.h, F, np,
                [&](uint32_t r) { return s_tok[r] * (d.k + 1) + s_slot[r]; }, smem, tab, tid,
                [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * H + row0 + tile * 16 + (ln & 15u)] =
                            s_wt[r] * sum0;
                });
        }
        b += nbat;
    }
}

// Sum of the k routed slots of one token at outputs o..o+3, in slot order; the loads of eight
// slots are issued together (k is a run-time value: a plain loop would wait for each in turn).
__device__ __forceinline__ float4 sum_routed_slots(const float* __restrict__ contrib_tok, uint32_t k, uint32_t H, uint32_t o)
{
    float4 r = float4{0.f, 0.f, 0.f, 0.f};
    for (uint32_t base = 0; base < k; base += 8) {
        float4 c[8];
#pragma unroll
        for (uint32_t i = 0; i < 8; i++)
            c[i] = base + i < k ? *(const float4*)(contrib_tok + (size_t)(base + i) * H + o) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) { r.x += c[i].x; r.y += c[i].y; r.z += c[i].z; r.w += c[i].w; } // + 0 is exact
    }
    return r;
}

// ---- fold: Y[t][o] = sum over the k routed slots in slot order + shared gate * shared slot ---------------
__global__ __launch_bounds__(256) void moe_fold_kernel(MoeWs ws, const qkk_sel* __restrict__ sel,
                                                       float* __restrict__ Y, MoeDims d, uint32_t N)
{
    const uint32_t quads = d.H / 4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)N * quads; i += (size_t)gridDim.x * 256) {
        const uint32_t t = (uint32_t)(i / quads), o = (uint32_t)(i % quads) * 4;
        float4 s = sum_routed_slots(ws.contrib + (size_t)t * (d.k + 1) * d.H, d.k, d.H, o);
        const float g = sel[t].w_shared;
        const float4 c = *(const float4*)(ws.contrib + ((size_t)t * (d.k + 1) + d.k) * d.H + o);
        s.x += g * c.x; s.y += g * c.y; s.z += g * c.z; s.w += g * c.w;
        *(float4*)(Y + (size_t)t * d.H + o) = s;
    }
}

// The fold with the layer tail behind it, one workgroup per token (n_embd = 2048: two quads per
// thread):  s = (resid + sum of the routed slots in slot order) + shared gate * shared slot, stored
// as the next residual, and xn = s * scale(s) * w with the NEXT layer's norm weight
// (reference shaders/add_rms3_grouped.comp:22-50).  resid may be S.
__global__ __launch_bounds__(256) void moe_fold_norm_kernel(MoeWs ws, const qkk_sel* __restrict__ sel, const float* resid,
                                                            const float* __restrict__ w, float* S, float* __restrict__ Xn,
                                                            MoeDims d, float eps)
{
    __shared__ float s_red[4];
    const uint32_t t = blockIdx.x;
    const float g = sel[t].w_shared;
    float4 v[2], gw[2]; // the norm weights are fetched with the row, not after the reduction
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) gw[j] = *(const float4*)(w + 4 * (threadIdx.x + 256u * j));
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t o = 4 * (threadIdx.x + 256u * j);
        const float4 r = sum_routed_slots(ws.contrib + (size_t)t * (d.k + 1) * d.H, d.k, d.H, o);
        const float4 a = *(const float4*)(resid + (size_t)t * d.H + o);
        const float4 c = *(const float4*)(ws.contrib + ((size_t)t * (d.k + 1) + d.k) * d.H + o);
        const float4 s = float4{(a.x + r.x) + g * c.x, (a.y + r.y) + g * c.y, (a.z + r.z) + g * c.z, (a.w + r.w) + g * c.w};
        *(float4*)(S + (size_t)t * d.H + o) = s;
        v[j] = s;
        ss += s.x * s.x;
        ss += s.y * s.y;
        ss += s.z * s.z;
        ss += s.w * s.w;
    }
    const float tot = block_sum4(ss, s_red);
    const float scale = 1.f / sqrtf(tot / (float)d.H + eps);
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t o = 4 * (threadIdx.x + 256u * j);
        *(float4*)(Xn + (size_t)t * d.H + o) = float4{v[j].x * scale * gw[j].x, v[j].y * scale * gw[j].y,
                                                      v[j].z * scale * gw[j].z, v[j].w * scale * gw[j].w};
    }
}

// ==== few rows (up to FUSED_MAX_ROWS): one gate/up and one down launch take the shared expert's and
// the routed experts' work together (a HIP graph runs the side stream's launches of so short a
// step one after the other, which costs more than it saves).
//
// Work of a launch = the shared expert's batches (token tiles x batches of weight rows, cost CS each)
// followed by the routed batches (active experts x batches, cost CR each).  Workgroup g of G takes
// the batches that start inside its equal share of the total cost: every workgroup gets the same
// work to within one batch whatever the number of active experts turns out to be (the host cannot
// know it), and its batches are consecutive, so they form at most a few runs of one expert's rows.
// ---- gate/up + SiLU --------------------------------------------------------------------------------
// n_embd = 2048: the eight waves take one 256-weight fragment each.  Routed experts: batches of
// one row tile of gate and of up (IQ3_XXS); shared expert (Q8_0): one row tile, gate and up in turns.
constexpr int FU_TG_R = 1, FU_TG_S = 1;
constexpr int FU_PB = 2; // partial buffers (2: one barrier per batch)
using FuGeoR = CoopGeom<QKK_IQ3_XXS, 8, 2, FU_TG_R, false, 1, FU_PB>;
using FuGeoS = CoopGeom<QKK_Q8_0, 8, 2, FU_TG_S, true, 1, FU_PB>;
constexpr uint32_t FU_LDS = FuGeoR::LDS_BYTES > FuGeoS::LDS_BYTES ? FuGeoR::LDS_BYTES : FuGeoS::LDS_BYTES;
constexpr uint32_t FU_CS = 3, FU_CR = 2; // a shared batch is two LDS steps, a routed one a single larger step

__global__ __launch_bounds__(CT) void moe_gateup_fused_kernel(const uint8_t* __restrict__ gate_exps,
                                                             const uint8_t* __restrict__ up_exps,
                                                             const uint8_t* __restrict__ gate_shexp,
                                                             const uint8_t* __restrict__ up_shexp,
                                                             const float* __restrict__ X, MoeWs ws, MoeDims d,
                                                             uint32_t N)
{
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t n_active = active_count(ws, d);
    const uint32_t tot_s = F / (16 * FuGeoS::BT), tot_r = F / (16 * FuGeoR::BT); // batches per token tile / expert
    const Share sh = my_share(blockIdx.x, gridDim.x, (N + 15) / 16 * tot_s, FU_CS, n_active * tot_r, FU_CR);
    const auto row_of = [&](uint32_t r) { return s_tok[r]; };

    for (uint32_t b = sh.s0; b < sh.s1;) { // shared expert: runs inside one token tile
        const uint32_t tile = b / tot_s, f0 = b % tot_s, nbat = min(tot_s - f0, sh.s1 - b);
        const uint32_t first = tile * 16u, np = min(16u, N - first), row0 = f0 * FuGeoS::BT * 16;
        __syncthreads(); // previous run fully consumed
        if (tid < 16) {
            s_tok[tid] = (uint32_t)tid < np ? first + tid : 0u;
            s_slot[tid] = d.k;
        }
        __syncthreads();
        coop_stream<QKK_Q8_0, 8, 2, FU_TG_S, true, false, 1, FU_PB>(gate_shexp + (size_t)row0 * FuGeoS::RB, up_shexp + (size_t)row0 * FuGeoS::RB, nbat, X, H, np, row_of, smem, tab, tid,
            [&](uint32_t t, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                const uint32_t r = 4 * (ln >> 4) + e;
                if (r < np)
                    ws.h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * F + row0 + t * 16 + (ln & 15u)] =
                        (sum0 / (1.f + expf(-sum0))) * sum1;
            });
        b += nbat;
    }
    for (uint32_t b = sh.r0; b < sh.r1;) { // routed: runs inside one active expert
        const uint32_t w = b / tot_r, f0 = b % tot_r, nbat = min(tot_r - f0, sh.r1 - b);
        const ActiveExpert a = active_expert(ws, w, d, N); // w < n_active
        const uint32_t row0 = f0 * FuGeoR::BT * 16;
        const size_t eo = ((size_t)a.expert * F + row0) * FuGeoR::RB;
        for (uint32_t t0 = 0; t0 < a.count; t0 += 16) {
            const uint32_t np = min(16u, a.count - t0);
            __syncthreads(); // previous tile fully consumed
            if (tid < 16) {
                uint32_t tok = 0, slot = 0;
                if ((uint32_t)tid < np) pair_at(ws, a.first + t0 + tid, d, N, tok, slot);
                s_tok[tid] = tok;
                s_slot[tid] = slot;
            }
            __syncthreads();
            coop_stream<QKK_IQ3_XXS, 8, 2, FU_TG_R, false, false, 1, FU_PB>(gate_exps + eo, up_exps + eo, nbat, X, H, np, row_of, smem, tab, tid,
                [&](uint32_t t, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * F + row0 + t * 16 + (ln & 15u)] =
                            (sum0 / (1.f + expf(-sum0))) * sum1;
                });
        }
        b += nbat;
    }
}

// ---- down: per-pair contributions -----------------------------------------------------------------
// contrib[(token*(k+1) + slot)*H + o] = weight * (D[o] . h[token][slot]); slot k = shared expert.
// K = F = 256*FB: FB waves split K, 8/FB tile groups split the batch's tiles.
template <int TYPE_DN, int FB>
struct DnGeoF {
    static constexpr int TG_R = TYPE_DN == QKK_Q6_K ? 1 : 2, TG_S = 1;
    using R = CoopGeom<TYPE_DN, FB, 1, TG_R>;
    using S = CoopGeom<QKK_Q8_0, FB, 1, TG_S>;
    static constexpr uint32_t LDS = R::LDS_BYTES > S::LDS_BYTES ? R::LDS_BYTES : S::LDS_BYTES;
    static constexpr uint32_t CS = 1, CR = TG_R; // cost of a batch ~ row tiles per wave
};

template <int TYPE_DN, int FB>
__global__ __launch_bounds__(CT) void moe_down_fused_kernel(const uint8_t* __restrict__ down_exps,
                                                           const uint8_t* __restrict__ down_shexp, MoeWs ws,
                                                           const qkk_sel* __restrict__ sel, MoeDims d, uint32_t N)
{
    using Geo = DnGeoF<TYPE_DN, FB>;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t n_active = active_count(ws, d);
    const uint32_t tot_s = H / (16 * Geo::S::BT), tot_r = H / (16 * Geo::R::BT);
    const Share sh = my_share(blockIdx.x, gridDim.x, (N + 15) / 16 * tot_s, Geo::CS, n_active * tot_r, Geo::CR);
    const auto row_of = [&](uint32_t r) { return s_tok[r] * (d.k + 1) + s_slot[r]; };

    for (uint32_t b = sh.s0; b < sh.s1;) {
        const uint32_t tile = b / tot_s, f0 = b % tot_s, nbat = min(tot_s - f0, sh.s1 - b);
        const uint32_t first = tile * 16u, np = min(16u, N - first), row0 = f0 * Geo::S::BT * 16;
        __syncthreads();
        if (tid < 16) {
            s_tok[tid] = (uint32_t)tid < np ? first + tid : 0u;
            s_slot[tid] = d.k;
            s_wt[tid] = (uint32_t)tid < np ? 1.f : 0.f; // the shared gate is applied by the fold
        }
        __syncthreads();
        coop_stream<QKK_Q8_0, FB, 1, Geo::TG_S, false, false>(down_shexp + (size_t)row0 * Geo::S::RB, nullptr, nbat, ws.h, F, np, row_of, smem, tab, tid,
            [&](uint32_t t, uint32_t ln, uint32_t e, float sum0, float, uint32_t) {
                const uint32_t r = 4 * (ln >> 4) + e;
                if (r < np)
                    ws.contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * H + row0 + t * 16 + (ln & 15u)] = s_wt[r] * sum0;
            });
        b += nbat;
    }
    for (uint32_t b = sh.r0; b < sh.r1;) {
        const uint32_t w = b / tot_r, f0 = b % tot_r, nbat = min(tot_r - f0, sh.r1 - b);
        const ActiveExpert a = active_expert(ws, w, d, N);
        const uint32_t row0 = f0 * Geo::R::BT * 16;
        const uint8_t* base = down_exps + ((size_t)a.expert * H + row0) * Geo::R::RB;
        for (uint32_t t0 = 0; t0 < a.count; t0 += 16) {
            const uint32_t np = min(16u, a.count - t0);
            __syncthreads();
            if (tid < 16) {
                uint32_t tok = 0, slot = 0;
                float wt = 0.f;
                if ((uint32_t)tid < np) {
                    pair_at(ws, a.first + t0 + tid, d, N, tok, slot);
                    wt = sel[tok].w[slot];
                }
                s_tok[tid] = tok; s_slot[tid] = slot; s_wt[tid] = wt;
            }
            __syncthreads();
            coop_stream<TYPE_DN, FB, 1, Geo::TG_R, false, false>(base, nullptr, nbat, ws.h, F, np, row_of, smem, tab, tid,
                [&](uint32_t t, uint32_t ln, uint32_t e, float sum0, float, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * H + row0 + t * 16 + (ln & 15u)] = s_wt[r] * sum0;
                });
        }
        b += nbat;
    }
}

// ---- host -----------------------------------------------------------------------------------------------
// workgroups of `fn` that fit a CU at once (registers, LDS): one or two; also raises its LDS limit
static uint32_t per_cu_of(const void* fn, uint32_t lds)
{
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    int n = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, CT, lds) != hipSuccess || n < 1) n = 1;
    return (uint32_t)std::min(n, 2);
}

template <int TYPE, int FB>
static void launch_down_fused(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d, uint32_t N,
                              hipStream_t st)
{
    using Geo = DnGeoF<TYPE, FB>;
    static const uint32_t per_cu = per_cu_of((const void*)moe_down_fused_kernel<TYPE, FB>, Geo::LDS);
    (void)per_cu;
    hipLaunchKernelGGL((moe_down_fused_kernel<TYPE, FB>), dim3(persistent_blocks() / 4), dim3(CT), Geo::LDS, st,
                       (const uint8_t*)L->down_exps, (const uint8_t*)L->down_shexp, ws, sel, d, N);
}

// Gate/up and down for few rows: shared and routed work in one launch each, one workgroup per CU.
void moe_mfma_launch_fused(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                           const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st)
{
    if (stages & QKK_STAGE_GATEUP) {
        static const uint32_t per_cu = per_cu_of((const void*)moe_gateup_fused_kernel, FU_LDS);
        (void)per_cu;
        hipLaunchKernelGGL(moe_gateup_fused_kernel, dim3(persistent_blocks() / 4), dim3(CT), FU_LDS, st,
                           (const uint8_t*)L->gate_exps, (const uint8_t*)L->up_exps, (const uint8_t*)L->gate_shexp,
                           (const uint8_t*)L->up_shexp, X, ws, d, N);
    }
    if (stages & QKK_STAGE_DOWN) {
        if (L->down_type == QKK_IQ4_XS) {
            if (d.F == 256) launch_down_fused<QKK_IQ4_XS, 1>(L, ws, sel, d, N, st);
            else if (d.F == 512) launch_down_fused<QKK_IQ4_XS, 2>(L, ws, sel, d, N, st);
            else launch_down_fused<QKK_IQ4_XS, 4>(L, ws, sel, d, N, st);
        } else {
            if (d.F == 256) launch_down_fused<QKK_Q6_K, 1>(L, ws, sel, d, N, st);
            else if (d.F == 512) launch_down_fused<QKK_Q6_K, 2>(L, ws, sel, d, N, st);
            else launch_down_fused<QKK_Q6_K, 4>(L, ws, sel, d, N, st);
        }
    }
}

// grid: what the device runs at once (per_cu workgroups per CU), no more than there are batches
template <bool SHARED>
static void launch_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, const MoeDims& d, uint32_t N,
                          uint32_t items, hipStream_t st)
{
    using Geo = GuGeo<SHARED>;
    static const uint32_t per_cu = per_cu_of((const void*)moe_gateup_mfma_kernel<SHARED>, Geo::LDS_BYTES);
    const uint32_t tot = d.F / (16 * Geo::BT);
    const uint32_t blocks = std::min(items * tot, per_cu * (persistent_blocks() / 4));
    hipLaunchKernelGGL(moe_gateup_mfma_kernel<SHARED>, dim3(blocks), dim3(CT), Geo::LDS_BYTES, st,
                       (const uint8_t*)(SHARED ? L->gate_shexp : L->gate_exps),
                       (const uint8_t*)(SHARED ? L->up_shexp : L->up_exps), X, ws, d, N);
}

template <int TYPE, int FB, bool SHARED>
static void launch_down(const void* W, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d, uint32_t N,
                        uint32_t items, hipStream_t st)
{
    using Geo = DnGeo<TYPE, FB>;
    static const uint32_t per_cu = per_cu_of((const void*)moe_down_mfma_kernel<TYPE, FB, SHARED>, Geo::LDS_BYTES);
    const uint32_t tot = d.H / (16 * Geo::BT);
    const uint32_t blocks = std::min(items * tot, per_cu * (persistent_blocks() / 4));
    hipLaunchKernelGGL((moe_down_mfma_kernel<TYPE, FB, SHARED>), dim3(blocks), dim3(CT), Geo::LDS_BYTES, st,
                       (const uint8_t*)W, ws, sel, d, N);
}

template <int TYPE, bool SHARED>
static void launch_down_f(const void* W, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d, uint32_t N,
                          uint32_t items, hipStream_t st)
{
    if (d.F == 256) launch_down<TYPE, 1, SHARED>(W, ws, sel, d, N, items, st);
    else if (d.F == 512) launch_down<TYPE, 2, SHARED>(W, ws, sel, d, N, items, st);
    else launch_down<TYPE, 4, SHARED>(W, ws, sel, d, N, items, st);
}

// The shared expert's launches of a step (side stream): gate/up, then down.
void moe_mfma_launch_shared(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                            const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st)
{
    const uint32_t tiles = (N + 15) / 16;
    if (stages & QKK_STAGE_GATEUP) launch_gateup<true>(L, X, ws, d, N, tiles, st);
    if (stages & QKK_STAGE_DOWN) launch_down_f<QKK_Q8_0, true>(L->down_shexp, ws, sel, d, N, tiles, st);
}

// The routed experts' launches of a step; the router record and the pair lists are in place.
void moe_mfma_launch_routed(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                            const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st)
{
    const uint32_t experts = (uint32_t)std::min<uint64_t>(d.E, (uint64_t)N * d.k); // upper bound of the active ones
    if (stages & QKK_STAGE_GATEUP) launch_gateup<false>(L, X, ws, d, N, experts, st);
    if (stages & QKK_STAGE_DOWN) {
        if (L->down_type == QKK_IQ4_XS) launch_down_f<QKK_IQ4_XS, false>(L->down_exps, ws, sel, d, N, experts, st);
        else launch_down_f<QKK_Q6_K, false>(L->down_exps, ws, sel, d, N, experts, st);
    }
}

// Sum of the k+1 slots (after both chains).
void moe_mfma_launch_fold(float* Y, const qkk_sel* sel, const MoeWs& ws, const MoeDims& d, uint32_t N, hipStream_t st)
{
    const uint32_t fb = (uint32_t)std::min<uint64_t>(((uint64_t)N * d.H / 4 + 255) / 256, persistent_blocks());
    hipLaunchKernelGGL(moe_fold_kernel, dim3(fb), dim3(256), 0, st, ws, sel, Y, d, N);
}

// The same with the residual add and the next layer's RMS norm (n_embd = 2048).
void moe_mfma_launch_fold_norm(const float* resid, const float* w_next, float eps, float* S, float* Xn,
                               const qkk_sel* sel, const MoeWs& ws, const MoeDims& d, uint32_t N, hipStream_t st)
{
    hipLaunchKernelGGL(moe_fold_norm_kernel, dim3(N), dim3(256), 0, st, ws, sel, resid, w_next, S, Xn, d, eps);
}

} // namespace qk
