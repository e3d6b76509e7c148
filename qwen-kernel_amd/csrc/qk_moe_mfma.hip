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

// Work items: first the shared expert's tiles of 16 consecutive tokens (one dense expert for
// every token: its items are the long ones, so they start first), then the routed experts with
// their pair lists.  Every item is cut into sub-items of `nb` batches of weight rows, so one
// expert's rows are streamed by several workgroups (each loads the activation rows itself).
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
// n_embd = 2048: the eight waves take one 256-weight fragment each.  Routed experts: batches of
// one row tile of gate and of up (IQ3_XXS); shared expert (Q8_0): one row tile, gate and up in turns.
constexpr int GU_TG_R = 1, GU_TG_S = 1;
constexpr int GU_PB = 2; // partial buffers (2: one barrier per batch)
using GuGeoR = CoopGeom<QKK_IQ3_XXS, 8, 2, GU_TG_R, false, 1, GU_PB>;
using GuGeoS = CoopGeom<QKK_Q8_0, 8, 2, GU_TG_S, true, 1, GU_PB>;
constexpr uint32_t GU_LDS = GuGeoR::LDS_BYTES > GuGeoS::LDS_BYTES ? GuGeoR::LDS_BYTES : GuGeoS::LDS_BYTES;

__global__ __launch_bounds__(CT) void moe_gateup_mfma_kernel(const uint8_t* __restrict__ gate_exps,
                                                             const uint8_t* __restrict__ up_exps,
                                                             const uint8_t* __restrict__ gate_shexp,
                                                             const uint8_t* __restrict__ up_shexp,
                                                             const float* __restrict__ X, MoeWs ws, MoeDims d,
                                                             uint32_t N, uint32_t nb_r, uint32_t nb_s)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t n_active = *ws.n_active;
    const uint32_t subs_sh = F / (16 * GuGeoS::BT * nb_s), subs = F / (16 * GuGeoR::BT * nb_r);
    const uint32_t n_items = item_count(n_active, N, subs_sh, subs);

    for (uint32_t w = blockIdx.x; w < n_items; w += gridDim.x) {
        const Item it = get_item(ws, w, subs_sh, subs, N);
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
            const auto row_of = [&](uint32_t r) { return s_tok[r]; };
            if (it.shared) {
                const uint32_t row0 = it.sub * nb_s * GuGeoS::BT * 16;
                coop_stream<QKK_Q8_0, 8, 2, GU_TG_S, true, false, 1, GU_PB>(gate_shexp + (size_t)row0 * GuGeoS::RB, up_shexp + (size_t)row0 * GuGeoS::RB, nb_s, X, H, np, row_of, smem, tab, tid,
                    [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                        const uint32_t r = 4 * (ln >> 4) + e;
                        if (r < np)
                            ws.h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * F + row0 + tile * 16 + (ln & 15u)] =
                                (sum0 / (1.f + expf(-sum0))) * sum1;
                    });
                break;
            }
            const uint32_t row0 = it.sub * nb_r * GuGeoR::BT * 16;
            const size_t eo = ((size_t)it.expert * F + row0) * GuGeoR::RB;
            coop_stream<QKK_IQ3_XXS, 8, 2, GU_TG_R, false, false, 1, GU_PB>(gate_exps + eo, up_exps + eo, nb_r, X, H, np, row_of, smem, tab, tid,
                [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.h[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * F + row0 + tile * 16 + (ln & 15u)] =
                            (sum0 / (1.f + expf(-sum0))) * sum1;
                });
        }
    }
}

// ---- down: per-pair contributions -----------------------------------------------------------------
// contrib[(token*(k+1) + slot)*H + o] = weight * (D[o] . h[token][slot]); slot k = shared expert.
// K = F = 256*FB: FB waves split K, 8/FB tile groups split the batch's tiles.
template <int TYPE_DN, int FB>
struct DnGeo {
    static constexpr int TG_R = TYPE_DN == QKK_Q6_K ? 1 : 2, TG_S = 1;
    using R = CoopGeom<TYPE_DN, FB, 1, TG_R>;
    using S = CoopGeom<QKK_Q8_0, FB, 1, TG_S>;
    static constexpr uint32_t LDS = R::LDS_BYTES > S::LDS_BYTES ? R::LDS_BYTES : S::LDS_BYTES;
};

template <int TYPE_DN, int FB>
__global__ __launch_bounds__(CT) void moe_down_mfma_kernel(const uint8_t* __restrict__ down_exps,
                                                           const uint8_t* __restrict__ down_shexp, MoeWs ws,
                                                           const qkk_sel* __restrict__ sel, MoeDims d, uint32_t N,
                                                           uint32_t nb_r, uint32_t nb_s)
{
    using Geo = DnGeo<TYPE_DN, FB>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x;
    const uint32_t F = d.F, H = d.H;
    fill_mfma_tables(tab, tid, CT);
    const uint32_t n_active = *ws.n_active;
    const uint32_t subs_sh = H / (16 * Geo::S::BT * nb_s), subs = H / (16 * Geo::R::BT * nb_r);
    const uint32_t n_items = item_count(n_active, N, subs_sh, subs);

    for (uint32_t w = blockIdx.x; w < n_items; w += gridDim.x) {
        const Item it = get_item(ws, w, subs_sh, subs, N);
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
            const auto row_of = [&](uint32_t r) { return s_tok[r] * (d.k + 1) + s_slot[r]; };
            if (it.shared) {
                const uint32_t row0 = it.sub * nb_s * Geo::S::BT * 16;
                coop_stream<QKK_Q8_0, FB, 1, Geo::TG_S, false, false>(down_shexp + (size_t)row0 * Geo::S::RB, nullptr, nb_s, ws.h, F, np, row_of, smem, tab, tid,
                    [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                        const uint32_t r = 4 * (ln >> 4) + e;
                        if (r < np)
                            ws.contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * H + row0 + tile * 16 + (ln & 15u)] =
                                s_wt[r] * sum0;
                    });
                break;
            }
            const uint32_t row0 = it.sub * nb_r * Geo::R::BT * 16;
            coop_stream<TYPE_DN, FB, 1, Geo::TG_R, false, false>(down_exps + ((size_t)it.expert * H + row0) * Geo::R::RB, nullptr, nb_r, ws.h, F, np, row_of, smem, tab, tid,
                [&](uint32_t tile, uint32_t ln, uint32_t e, float sum0, float sum1, uint32_t) {
                    const uint32_t r = 4 * (ln >> 4) + e;
                    if (r < np)
                        ws.contrib[((size_t)s_tok[r] * (d.k + 1) + s_slot[r]) * H + row0 + tile * 16 + (ln & 15u)] =
                            s_wt[r] * sum0;
                });
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
static void set_lds_attr(const void* fn, uint32_t bytes)
{
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// batches per sub-item: the largest power of two <= total that still gives every CU about two items
static uint32_t pick_nb(uint32_t total_batches, uint32_t experts)
{
    uint32_t nb = total_batches;
    while (nb > 1 && (uint64_t)experts * (total_batches / nb) < 2ull * persistent_blocks() / 4) nb /= 2;
    return nb;
}

template <int TYPE, int FB>
static void launch_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d, uint32_t N,
                        uint32_t experts, hipStream_t st)
{
    using Geo = DnGeo<TYPE, FB>;
    static bool once = (set_lds_attr((const void*)moe_down_mfma_kernel<TYPE, FB>, Geo::LDS), true);
    (void)once;
    const uint32_t tot_r = d.H / (16 * Geo::R::BT), tot_s = d.H / (16 * Geo::S::BT);
    const uint32_t nb_r = pick_nb(tot_r, experts), nb_s = std::min(tot_s, std::max(1u, nb_r * Geo::R::BT / Geo::S::BT / 2));
    const uint32_t items = experts * (tot_r / nb_r) + (N + 15) / 16 * (tot_s / nb_s);
    const uint32_t blocks = std::min(items, persistent_blocks() / 4);
    hipLaunchKernelGGL((moe_down_mfma_kernel<TYPE, FB>), dim3(blocks), dim3(CT), Geo::LDS, st,
                       (const uint8_t*)L->down_exps, (const uint8_t*)L->down_shexp, ws, sel, d, N, nb_r, nb_s);
}

// Gate/up, down and fold for N >= 2 rows; the router record and the pair lists are in place.
void moe_mfma_launch(const qkk_moe_layer* L, const float* X, float* Y, const qkk_sel* sel, const MoeWs& ws,
                     const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st)
{
    const uint32_t experts = (uint32_t)std::min<uint64_t>(d.E, (uint64_t)N * d.k); // upper bound of the active ones
    if (stages & QKK_STAGE_GATEUP) {
        static const uint32_t per_cu = [] { // workgroups that fit a CU at once (registers, LDS)
            set_lds_attr((const void*)moe_gateup_mfma_kernel, GU_LDS);
            int n = 1;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)moe_gateup_mfma_kernel, CT, GU_LDS) != hipSuccess || n < 1)
                n = 1;
            return (uint32_t)std::min(n, 2);
        }();
        const uint32_t tot_r = d.F / (16 * GuGeoR::BT), tot_s = d.F / (16 * GuGeoS::BT);
        const uint32_t nb_r = pick_nb(tot_r, experts), nb_s = std::min(tot_s, std::max(1u, nb_r * GuGeoR::BT / GuGeoS::BT / 2));
        const uint32_t items = experts * (tot_r / nb_r) + (N + 15) / 16 * (tot_s / nb_s);
        const uint32_t blocks = std::min(items, per_cu * (persistent_blocks() / 4));
        hipLaunchKernelGGL(moe_gateup_mfma_kernel, dim3(blocks), dim3(CT), GU_LDS, st, (const uint8_t*)L->gate_exps,
                           (const uint8_t*)L->up_exps, (const uint8_t*)L->gate_shexp, (const uint8_t*)L->up_shexp, X, ws, d,
                           N, nb_r, nb_s);
    }
    if (stages & QKK_STAGE_DOWN) {
        if (L->down_type == QKK_IQ4_XS) {
            if (d.F == 256) launch_down<QKK_IQ4_XS, 1>(L, ws, sel, d, N, experts, st);
            else if (d.F == 512) launch_down<QKK_IQ4_XS, 2>(L, ws, sel, d, N, experts, st);
            else launch_down<QKK_IQ4_XS, 4>(L, ws, sel, d, N, experts, st);
        } else {
            if (d.F == 256) launch_down<QKK_Q6_K, 1>(L, ws, sel, d, N, experts, st);
            else if (d.F == 512) launch_down<QKK_Q6_K, 2>(L, ws, sel, d, N, experts, st);
            else launch_down<QKK_Q6_K, 4>(L, ws, sel, d, N, experts, st);
        }
        const uint32_t fb = (uint32_t)std::min<uint64_t>(((uint64_t)N * d.H / 4 + 255) / 256, persistent_blocks());
        hipLaunchKernelGGL(moe_fold_kernel, dim3(fb), dim3(256), 0, st, ws, Y, d, N);
    }
}

} // namespace qk
