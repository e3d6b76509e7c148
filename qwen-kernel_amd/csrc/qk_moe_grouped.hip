// qk_moe_grouped.hip -- expert-major MoE step for several tokens (decode slots or a prefill
// chunk) on VALU.
//
// Each expert picked by at least one token is visited once: its gate/up rows and its down
// rows are fetched once and applied to every (token, pick) pair routed to it, so the
// expert's bytes cross HBM once however many tokens share it
// (the expert-major order of reference shaders/moe_gateup_iq3_grouped.comp:30-114 and
// moe_down_iq4_grouped.comp:24-75, driven by the pair lists of moe_group_pairs.comp).
// Launches: route (router logits, shared gate/up, and -- in the block that finishes last --
// top-k selection and pair grouping), grouped gate/up, grouped down into per-pair
// contributions, fold (+ shared down).
#include "qk_moe_common.h"

#include <algorithm>

namespace qk {

constexpr uint32_t SELECT_INLINE_MAX = 64; // up to this many tokens the route launch also selects

// ---- selection + grouping by one workgroup of NW waves ------------------------------------
template <int NW>
__device__ static void select_and_group(const MoeWs& ws, qkk_sel* __restrict__ sel, MoeDims d, uint32_t N,
                                        float* s_log, uint32_t* s_cnt, uint32_t* s_cur)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* my_log = s_log + (size_t)wave * (QKK_MAX_EXPERTS + 8);
    for (uint32_t t = wave; t < N; t += NW) {
        // the caller's acquire fence precedes this: plain loads, all issued before the first use
        const float* gl = ws.logits + (size_t)t * lstride(d.E);
        float lv[QKK_MAX_EXPERTS / 64 + 1];
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            lv[i] = (uint32_t)(lane + 64 * i) <= d.E ? gl[lane + 64 * i] : 0.f;
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            if ((uint32_t)(lane + 64 * i) <= d.E) my_log[lane + 64 * i] = lv[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        select_wave(my_log, d.E, d.k, &sel[t]);
        if (lane == 0) sel[t].w_shared = 1.f / (1.f + expf(-my_log[d.E]));
        __builtin_amdgcn_wave_barrier();
    }
    for (uint32_t e = threadIdx.x; e <= QKK_MAX_EXPERTS; e += NW * 64) s_cnt[e] = 0;
    __threadfence_block();
    __syncthreads();
    const uint32_t np = N * d.k;
    const volatile qkk_sel* vs = sel;
    for (uint32_t p = threadIdx.x; p < np; p += NW * 64)
        atomicAdd(&s_cnt[min(vs[p / d.k].ids[p % d.k], d.E - 1)], 1u);
    __syncthreads();
    // exclusive scan over the experts of (pair count, "has pairs" flag), packed count | flag<<20
    // (count <= 4096*16 < 2^20): Hillis-Steele in LDS, two experts per thread when NW = 4
    constexpr uint32_t PER = (QKK_MAX_EXPERTS + NW * 64 - 1) / (NW * 64);
    uint32_t mine[PER], incl[PER];
#pragma unroll
    for (uint32_t j = 0; j < PER; j++) {
        const uint32_t e = threadIdx.x + j * NW * 64;
        const uint32_t c = e < d.E ? s_cnt[e] : 0u;
        mine[j] = c | (c ? 1u << 20 : 0u);
        incl[j] = mine[j];
    }
    for (uint32_t step = 1; step < QKK_MAX_EXPERTS; step <<= 1) {
#pragma unroll
        for (uint32_t j = 0; j < PER; j++) {
            const uint32_t e = threadIdx.x + j * NW * 64;
            if (e < QKK_MAX_EXPERTS) s_cur[e] = incl[j];
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < PER; j++) {
            const uint32_t e = threadIdx.x + j * NW * 64;
            if (e < QKK_MAX_EXPERTS && e >= step) incl[j] += s_cur[e - step];
        }
        __syncthreads();
    }
#pragma unroll
    for (uint32_t j = 0; j < PER; j++) {
        const uint32_t e = threadIdx.x + j * NW * 64;
        if (e >= QKK_MAX_EXPERTS) continue;
        const uint32_t excl = incl[j] - mine[j];
        const uint32_t off = excl & 0xFFFFFu, rank = excl >> 20, c = mine[j] & 0xFFFFFu;
        s_cur[e] = off;
        if (e < d.E) {
            ws.offsets[e] = off;
            if (c) {
                ActiveExpert a{e, off, c, 0};
                ws.active[rank] = a;
            }
        }
        if (e == d.E - 1) {
            ws.offsets[d.E] = off + c;
            *ws.n_active = rank + (c ? 1u : 0u);
        }
    }
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < np; p += NW * 64) {
        const uint32_t t = p / d.k, s = p % d.k;
        const uint32_t e = min(vs[t].ids[s], d.E - 1);
        ws.pairs[atomicAdd(&s_cur[e], 1u)] = (t << 4) | s;
    }
}

// ---- launch 1: router + shared gate/up for N tokens ----------------------------------------
// One wave per task = (router row | shared row pair) x (group of TG tokens).  All loads of a
// task -- its weights and the TG activation slices -- are issued together: one memory round
// trip per task.  Weights are re-read once per token group (from L2 after the first).
template <int NCH>
__global__ __launch_bounds__(512) void moe_route_multi_kernel(const float* __restrict__ gate_inp,
                                                              const float* __restrict__ gate_inp_shexp,
                                                              const uint8_t* __restrict__ gate_shexp,
                                                              const uint8_t* __restrict__ up_shexp,
                                                              const float* __restrict__ X, MoeWs ws,
                                                              qkk_sel* __restrict__ sel, MoeDims d, uint32_t N,
                                                              uint32_t select_here)
{
    constexpr int P = NCH / 8;
    constexpr int TG = NCH <= 8 ? 4 : 2; // tokens per task
    constexpr int NW = 8;                // waves per block
    __shared__ uint32_t s_last;
    __shared__ float s_log[NW * (QKK_MAX_EXPERTS + 8)];
    __shared__ uint32_t s_cnt[QKK_MAX_EXPERTS + 1], s_cur[QKK_MAX_EXPERTS + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_dense = d.E + 1, n_rows = n_dense + d.F;
    const uint32_t q8_row = d.H / 32 * Q8_0_BYTES;
    const uint32_t task = blockIdx.x * NW + wave;
    const uint32_t t = task % n_rows, t0 = (task / n_rows) * TG;
    const uint32_t LS = lstride(d.E);

    if (t0 < N && t < n_dense) {
        const float4* row = (const float4*)(t < d.E ? gate_inp + (size_t)t * d.H : gate_inp_shexp);
        float4 w[NCH], xx[TG][NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
#pragma unroll
        for (int j = 0; j < TG; j++) {
            const float4* xv = (const float4*)(X + (size_t)min(t0 + j, N - 1) * d.H);
#pragma unroll
            for (int i = 0; i < NCH; i++) xx[j][i] = xv[lane + 64 * i];
        }
#pragma unroll
        for (int j = 0; j < TG; j++) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                a0 += w[i].x * xx[j][i].x + w[i].y * xx[j][i].y;
                a1 += w[i].z * xx[j][i].z + w[i].w * xx[j][i].w;
            }
            const float s = wave_sum(a0 + a1);
            if (lane == 0 && t0 + j < N) publish(&ws.logits[(size_t)(t0 + j) * LS + t], s);
        }
    } else if (t0 < N) {
        const uint32_t r = t - n_dense;
        LaneW<QKK_Q8_0> wg[P], wu[P];
        XSlice xs[TG][P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            wg[p].load(gate_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
            wu[p].load(up_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
        }
#pragma unroll
        for (int j = 0; j < TG; j++)
#pragma unroll
            for (int p = 0; p < P; p++)
                load_xslice<QKK_Q8_0>(xs[j][p], X + (size_t)min(t0 + j, N - 1) * d.H + p * 2048, lane);
#pragma unroll
        for (int j = 0; j < TG; j++) {
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int p = 0; p < P; p++) {
                wg[p].touch();
                wu[p].touch();
                g += wg[p].dot(xs[j][p], nullptr, nullptr, lane);
                u += wu[p].dot(xs[j][p], nullptr, nullptr, lane);
            }
            g = wave_sum(g);
            u = wave_sum(u);
            if (lane == 0 && t0 + j < N)
                ws.h[((size_t)(t0 + j) * (d.k + 1) + d.k) * d.F + r] = (g / (1.f + expf(-g))) * u;
        }
    }
    if (!select_here) return;

    // only the logits are read back inside this launch (by the selecting workgroup); the
    // shared-expert h is read by the next launch
    __syncthreads();
    if (threadIdx.x == 0) s_last = arrive_last(&ws.counter[0], gridDim.x) ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        select_and_group<NW>(ws, sel, d, N, s_log, s_cnt, s_cur);
        if (threadIdx.x == 0) ws.counter[0] = 0u;
    }
}

// Selection + grouping as a launch of its own (many tokens).
__global__ __launch_bounds__(1024) void moe_select_group_kernel(MoeWs ws, qkk_sel* __restrict__ sel, MoeDims d,
                                                                uint32_t N)
{
    __shared__ float s_log[16 * (QKK_MAX_EXPERTS + 8)];
    __shared__ uint32_t s_cnt[QKK_MAX_EXPERTS + 1], s_cur[QKK_MAX_EXPERTS + 1];
    select_and_group<16>(ws, sel, d, N, s_log, s_cnt, s_cur);
}

// ---- launch 2: expert-major gate/up -----------------------------------------------------------
template <int TYPE, int PASSES, int RIF>
__global__ __launch_bounds__(256) void moe_gateup_grouped_kernel(const uint8_t* __restrict__ gate_exps,
                                                                 const uint8_t* __restrict__ up_exps,
                                                                 const float* __restrict__ X, MoeWs ws, MoeDims d)
{
    __shared__ IqTables tab;
    fill_iq_tables(tab, g_iq3xxs_grid, threadIdx.x, 256);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row_bytes = (uint32_t)qkk_row_bytes_dev<TYPE>(d.H);
    const uint32_t pass_bytes = row_bytes / PASSES;
    const uint32_t groups = (d.F + RIF - 1) / RIF;
    const uint32_t n_tasks = *ws.n_active * groups;
    for (uint32_t task = blockIdx.x * 4 + wave; task < n_tasks; task += gridDim.x * 4) {
        const ActiveExpert a = ws.active[task / groups];
        const uint32_t r0 = (task % groups) * RIF;
        const uint8_t* gbase = gate_exps + ((size_t)a.expert * d.F) * row_bytes;
        const uint8_t* ubase = up_exps + ((size_t)a.expert * d.F) * row_bytes;
        LaneW<TYPE> wg[RIF][PASSES], wu[RIF][PASSES];
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            const uint32_t r = min(r0 + i, d.F - 1);
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                wg[i][p].load(gbase + (size_t)r * row_bytes + (size_t)p * pass_bytes, lane);
                wu[i][p].load(ubase + (size_t)r * row_bytes + (size_t)p * pass_bytes, lane);
            }
        }
        for (uint32_t q = 0; q < a.count; q++) {
            const uint32_t pr = ws.pairs[a.first + q];
            const uint32_t tok = pr >> 4, s = pr & 15u;
            XSlice xs[PASSES];
#pragma unroll
            for (int p = 0; p < PASSES; p++) load_xslice<TYPE>(xs[p], X + (size_t)tok * d.H + p * 2048, lane);
#pragma unroll
            for (int i = 0; i < RIF; i++) {
#pragma unroll
                for (int p = 0; p < PASSES; p++) {
                    wg[i][p].touch();
                    wu[i][p].touch();
                }
                float g = 0.f, u = 0.f;
#pragma unroll
                for (int p = 0; p < PASSES; p++) {
                    g += wg[i][p].dot(xs[p], nullptr, &tab, lane);
                    u += wu[i][p].dot(xs[p], nullptr, &tab, lane);
                }
                g = wave_sum(g);
                u = wave_sum(u);
                if (lane == 0 && r0 + i < d.F)
                    ws.h[((size_t)tok * (d.k + 1) + s) * d.F + r0 + i] = (g / (1.f + expf(-g))) * u;
            }
        }
    }
}

// ---- launch 3: expert-major down into per-pair contributions -----------------------------------
// contrib[(token*k + pick)*H + o] = w[token][pick] * (D_expert[o] . h[token][pick])
// (reference shaders/moe_down_iq4_grouped.comp:67-72).  F = 32*LPR.
template <int TYPE, int LPR, int RIF>
__global__ __launch_bounds__(256) void moe_down_grouped_kernel(const uint8_t* __restrict__ down_exps, MoeWs ws,
                                                               const qkk_sel* __restrict__ sel, MoeDims d)
{
    __shared__ IqTables tab;
    fill_iq_tables(tab, g_iq3xxs_grid, threadIdx.x, 256);
    __syncthreads();
    constexpr int GROUPS = WAVE / LPR;
    constexpr uint32_t CHUNK = GROUPS * RIF;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const uint32_t row_bytes = (uint32_t)qkk_row_bytes_dev<TYPE>(d.F);
    const uint32_t chunks = (d.H + CHUNK - 1) / CHUNK;
    const uint32_t n_tasks = *ws.n_active * chunks;
    for (uint32_t task = blockIdx.x * 4 + wave; task < n_tasks; task += gridDim.x * 4) {
        const ActiveExpert a = ws.active[task / chunks];
        const uint32_t o0 = (task % chunks) * CHUNK;
        const uint8_t* base = down_exps + (size_t)a.expert * d.H * row_bytes;
        LaneW<TYPE> w[RIF];
#pragma unroll
        for (int i = 0; i < RIF; i++)
            w[i].load(base + (size_t)min(o0 + i * GROUPS + grp, d.H - 1) * row_bytes, lir);
        for (uint32_t q = 0; q < a.count; q++) {
            const uint32_t pr = ws.pairs[a.first + q];
            const uint32_t tok = pr >> 4, s = pr & 15u;
            const float wt = sel[tok].w[s];
            XSlice hs;
            load_xslice<TYPE>(hs, ws.h + ((size_t)tok * (d.k + 1) + s) * d.F, lir);
            float hsum[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                float v = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) v += hs.v[c * 8 + i];
                hsum[c] = v;
            }
#pragma unroll
            for (int i = 0; i < RIF; i++) {
                float acc = wt * w[i].dot(hs, hsum, &tab, lir);
                acc = lanes_sum<LPR>(acc);
                const uint32_t o = o0 + i * GROUPS + grp;
                if (lir == 0 && o < d.H) ws.contrib[((size_t)tok * d.k + s) * d.H + o] = acc;
            }
        }
    }
}

// ---- launch 4: fold the contributions, add the shared expert -------------------------------------
// Y[t][o] = sum_s contrib[t][s][o] + w_shared[t] * (Ds[o] . h[t][k]); the shared down rows stay
// in registers while the wave walks the tokens.
template <int LPR, int RIF>
__global__ __launch_bounds__(256) void moe_fold_shared_kernel(const uint8_t* __restrict__ down_shexp, MoeWs ws,
                                                              const qkk_sel* __restrict__ sel,
                                                              float* __restrict__ Y, MoeDims d, uint32_t N)
{
    constexpr int GROUPS = WAVE / LPR;
    constexpr uint32_t CHUNK = GROUPS * RIF;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const uint32_t q8_row = d.F / 32 * Q8_0_BYTES;
    for (uint32_t o0 = (blockIdx.x * 4 + wave) * CHUNK; o0 < d.H; o0 += gridDim.x * 4 * CHUNK) {
        LaneW<QKK_Q8_0> w[RIF];
#pragma unroll
        for (int i = 0; i < RIF; i++)
            w[i].load(down_shexp + (size_t)min(o0 + i * GROUPS + grp, d.H - 1) * q8_row, lir);
        for (uint32_t t = 0; t < N; t++) {
            XSlice hs;
            load_xslice<QKK_Q8_0>(hs, ws.h + ((size_t)t * (d.k + 1) + d.k) * d.F, lir);
            const float wsh = sel[t].w_shared;
            float part[RIF];
#pragma unroll
            for (int i = 0; i < RIF; i++) {
                const uint32_t o = min(o0 + i * GROUPS + grp, d.H - 1);
                float c = 0.f;
                for (uint32_t s = lir; s < d.k; s += LPR) c += ws.contrib[((size_t)t * d.k + s) * d.H + o];
                part[i] = c;
            }
#pragma unroll
            for (int i = 0; i < RIF; i++) {
                float acc = wsh * w[i].dot(hs, nullptr, nullptr, lir) + part[i];
                acc = lanes_sum<LPR>(acc);
                const uint32_t o = o0 + i * GROUPS + grp;
                if (lir == 0 && o < d.H) Y[(size_t)t * d.H + o] = acc;
            }
        }
    }
}

template <int TYPE, int LPR>
static void launch_down_grouped(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, const MoeDims& d,
                                uint32_t max_active, hipStream_t st)
{
    constexpr int RIF = 4;
    const uint32_t chunks = (d.H + (64 / LPR) * RIF - 1) / ((64 / LPR) * RIF);
    const uint32_t blocks = std::min((max_active * chunks + 3) / 4, persistent_blocks());
    hipLaunchKernelGGL((moe_down_grouped_kernel<TYPE, LPR, RIF>), dim3(blocks), dim3(256), 0, st,
                       (const uint8_t*)L->down_exps, ws, sel, d);
}

template <int LPR>
static void launch_fold(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y, const MoeDims& d,
                        uint32_t N, hipStream_t st)
{
    constexpr int RIF = 2;
    const uint32_t chunks = (d.H + (64 / LPR) * RIF - 1) / ((64 / LPR) * RIF);
    hipLaunchKernelGGL((moe_fold_shared_kernel<LPR, RIF>), dim3((chunks + 3) / 4), dim3(256), 0, st,
                       (const uint8_t*)L->down_shexp, ws, sel, Y, d, N);
}

// Host entry of the grouped path (arguments already validated).
int moe_grouped_launch(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                       uint32_t N, uint32_t stages, hipStream_t st)
{
    const MoeDims d{L->n_embd, L->n_ff, L->n_expert, L->n_used};
    const MoeWs ws = ws_carve(workspace, d, N);
    const uint32_t t1 = d.E + 1 + d.F;
    const uint32_t inline_sel = N <= SELECT_INLINE_MAX ? 1u : 0u;
    const uint8_t* gs = (const uint8_t*)L->gate_shexp;
    const uint8_t* us = (const uint8_t*)L->up_shexp;
    if (!(stages & QKK_STAGE_ROUTE)) {
    } else if (d.H == 2048) {
        const uint32_t tasks = t1 * ((N + 3) / 4);
        hipLaunchKernelGGL(moe_route_multi_kernel<8>, dim3((tasks + 7) / 8), dim3(512), 0, st, L->gate_inp,
                           L->gate_inp_shexp, gs, us, X, ws, sel, d, N, inline_sel);
    } else {
        const uint32_t tasks = t1 * ((N + 1) / 2);
        hipLaunchKernelGGL(moe_route_multi_kernel<16>, dim3((tasks + 7) / 8), dim3(512), 0, st, L->gate_inp,
                           L->gate_inp_shexp, gs, us, X, ws, sel, d, N, inline_sel);
    }
    if ((stages & QKK_STAGE_ROUTE) && !inline_sel) hipLaunchKernelGGL(moe_select_group_kernel, dim3(1), dim3(1024), 0, st, ws, sel, d, N);

    const uint32_t max_active = std::min<uint64_t>(d.E, (uint64_t)N * d.k);
    const uint8_t* ge = (const uint8_t*)L->gate_exps;
    const uint8_t* ue = (const uint8_t*)L->up_exps;
    if (!(stages & QKK_STAGE_GATEUP)) {
    } else if (d.H == 2048) {
        constexpr int RIF = 4;
        const uint32_t blocks = std::min((max_active * ((d.F + RIF - 1) / RIF) + 3) / 4, persistent_blocks());
        hipLaunchKernelGGL((moe_gateup_grouped_kernel<QKK_IQ3_XXS, 1, RIF>), dim3(blocks), dim3(256), 0, st, ge, ue,
                           X, ws, d);
    } else {
        constexpr int RIF = 2;
        const uint32_t blocks = std::min((max_active * ((d.F + RIF - 1) / RIF) + 3) / 4, persistent_blocks());
        hipLaunchKernelGGL((moe_gateup_grouped_kernel<QKK_IQ3_XXS, 2, RIF>), dim3(blocks), dim3(256), 0, st, ge, ue,
                           X, ws, d);
    }
    if (!(stages & QKK_STAGE_DOWN)) return check_launch("moe grouped path");
    if (L->down_type == QKK_IQ4_XS) {
        if (d.F == 512) launch_down_grouped<QKK_IQ4_XS, 16>(L, ws, sel, d, max_active, st);
        else if (d.F == 256) launch_down_grouped<QKK_IQ4_XS, 8>(L, ws, sel, d, max_active, st);
        else launch_down_grouped<QKK_IQ4_XS, 32>(L, ws, sel, d, max_active, st);
    } else {
        if (d.F == 512) launch_down_grouped<QKK_Q6_K, 16>(L, ws, sel, d, max_active, st);
        else if (d.F == 256) launch_down_grouped<QKK_Q6_K, 8>(L, ws, sel, d, max_active, st);
        else launch_down_grouped<QKK_Q6_K, 32>(L, ws, sel, d, max_active, st);
    }
    if (d.F == 512) launch_fold<16>(L, ws, sel, Y, d, N, st);
    else if (d.F == 256) launch_fold<8>(L, ws, sel, Y, d, N, st);
    else launch_fold<32>(L, ws, sel, Y, d, N, st);
    return check_launch("moe grouped path");
}

} // namespace qk
