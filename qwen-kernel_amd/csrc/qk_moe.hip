// qk_moe.hip -- fused Qwen3-MoE decode step for gfx950.
//
// One activation row, three launches per step:
//   1. route:   router logits (F32 rows) + shared-expert gate dot + shared gate/up (Q8_0).
//   2. gate/up: every workgroup picks the top-n_used experts from the logits, then the routed
//               IQ3_XXS gate and up rows of the picks, SiLU gating -> h; writes the router record.
//   3. down:    routed down rows (IQ4_XS or Q6_K) weighted by the router, shared down row
//               (Q8_0) weighted by the sigmoid gate, summed into y.
// Inside a HIP graph a launch costs about 1.7 us whatever it does and a cold read of a few MB adds
// about 1 us, while a device-wide barrier inside a kernel measured 5 us: so the step is three
// launches, each arranged as at most two dependent round trips to memory.  Block rows are streamed
// as 16-byte pieces through a wave-private LDS area (qk_stream.h): with per-lane loads of the
// misaligned block fields the address unit of the CU, not memory, set the pace (the picked experts'
// 6.4 MB took 4.5 us to arrive).  Several rows go through the expert-major path in
// qk_moe_grouped.hip.
#include "qk_moe_common.h"
#include "qk_stream.h"

#include <mutex>
#include <stdlib.h>

namespace qk {

template <bool ON>
struct NormArg {
    const float* w; // RMS-norm weights of the row
    float eps;
};
template <>
struct NormArg<false> {};

// ADD: the row is x + mix (a mixer's output on top of the residual); the first workgroup of the row
// also stores the sum to `sum`, a buffer of its own, for the launches behind this one.
template <bool ON>
struct AddArg {
    const float* mix;
    float* sum;
};
template <>
struct AddArg<false> {};

// Sum over a workgroup of NW waves in wave order; every thread returns the same bits.
template <int NW>
__device__ __forceinline__ float block_sum_waves(float v, float* s_red)
{
    const float w = wave_sum(v);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = w;
    __syncthreads();
    float t = s_red[0];
#pragma unroll
    for (int i = 1; i < NW; i++) t += s_red[i];
    return t;
}

// The workgroup (NT threads) forms x * nw once, in LDS, and returns 1/sqrt(mean(x^2) + eps): a dot
// product against the normalised row is that factor times the dot product against x * nw, so the
// callers run on x * nw and scale their sums.  (A wave that fetched x and nw for itself made the
// launch 1.7 us longer: three 8 KB rows per wave through the L1 instead of two.)  ADD as above.
// The barrier inside the block sum also publishes s_x.
template <int NT, int NQ /* float4s of the row */, bool ADD>
__device__ __forceinline__ float stage_normed_row(const float* __restrict__ x, const float* __restrict__ nw, float eps,
                                                  float* s_x, float* s_red, const AddArg<ADD>& aa, bool store_sum)
{
    constexpr int NV = (NQ + NT - 1) / NT;
    float4 xv[NV], nv[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const uint32_t q = min(threadIdx.x + NT * i, (uint32_t)NQ - 1);
        xv[i] = ((const float4*)x)[q];
        nv[i] = ((const float4*)nw)[q];
    }
    if constexpr (ADD) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const uint32_t q = min(threadIdx.x + NT * i, (uint32_t)NQ - 1);
            const float4 m = ((const float4*)aa.mix)[q];
            xv[i] = float4{xv[i].x + m.x, xv[i].y + m.y, xv[i].z + m.z, xv[i].w + m.w};
            if (store_sum && threadIdx.x + NT * i < NQ) ((float4*)aa.sum)[q] = xv[i];
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        if (threadIdx.x + NT * i < NQ) {
            ss += (xv[i].x * xv[i].x + xv[i].y * xv[i].y) + (xv[i].z * xv[i].z + xv[i].w * xv[i].w);
            ((float4*)s_x)[threadIdx.x + NT * i] =
                float4{xv[i].x * nv[i].x, xv[i].y * nv[i].y, xv[i].z * nv[i].z, xv[i].w * nv[i].w};
        }
    }
    return 1.f / sqrtf(block_sum_waves<NT / 64>(ss, s_red) / (float)(4 * NQ) + eps);
}

// ---- launch 1: router logits + shared gate/up ---------------------------------------------
// One wave per task, no loop: tasks [0, E] are F32 rows (row E = the shared gate row), tasks after
// that are shared-expert gate/up row pairs (Q8_0, both rows staged through LDS).  Every load of a
// task is issued before its arithmetic, so a task costs one memory round trip.  Three waves per
// workgroup: E + 1 + F = 769 tasks make 257 workgroups, three tasks on every CU (four waves per
// workgroup made 193 and left a quarter of the CUs idle).  H = 256*NCH.
// ROWS: blockIdx.y is the activation row (slot); every row runs the one-row launch on its own part
// of x and of the workspace -- for a few rows, which hardly ever pick the same expert, this beats
// the expert-major path, and a row's result does not depend on its company.
// MODE 0: x is the (normalised) activation row.  MODE 1: x is the un-normalised residual row, the
// RMS norm with weights na.w runs in front (stage_normed_row).  MODE 2: the row is x + mix.
constexpr int ROUTE_WAVES = 3;

template <int NCH, bool ROWS, int MODE>
__global__ __launch_bounds__(64 * ROUTE_WAVES) void moe_route_kernel(const float* __restrict__ gate_inp,
                                                        const float* __restrict__ gate_inp_shexp,
                                                        const uint8_t* __restrict__ gate_shexp,
                                                        const uint8_t* __restrict__ up_shexp,
                                                        const float* __restrict__ x, MoeWs ws, MoeDims d,
                                                        NormArg<MODE != 0> na, AddArg<MODE == 2> aa)
{
    if constexpr (MODE == 2) {
        if constexpr (ROWS) {
            aa.mix += (size_t)blockIdx.y * d.H;
            aa.sum += (size_t)blockIdx.y * d.H;
        }
    }
    if constexpr (ROWS) {
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
    }
    constexpr int P = NCH / 8;                          // 2048-weight passes per Q8_0 row
    constexpr uint32_t Q8ROW = 64 * P * Q8_0_BYTES;     // bytes of one shared-expert row
    constexpr uint32_t NPIECE = 2 * Q8ROW / 16;         // the gate row, then the up row
    constexpr int NP = (NPIECE + 63) / 64;
    __shared__ __attribute__((aligned(16))) uint8_t s_stage[ROUTE_WAVES][WaveStage<NP>::AREA + 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_dense = d.E + 1, n_tasks = n_dense + d.F;
    const uint32_t t = blockIdx.x * ROUTE_WAVES + wave;

    // the task's weights first: they are in flight while x arrives
    const bool dense = t < n_dense, shared = !dense && t < n_tasks;
    float4 w[NCH];
    WaveStage<NP> st;
    if (dense) {
        const float4* row = (const float4*)(t < d.E ? gate_inp + (size_t)t * d.H : gate_inp_shexp);
#pragma unroll
        for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
    } else if (shared) {
        const uint8_t* g = gate_shexp + (size_t)(t - n_dense) * Q8ROW;
        const uint8_t* u = up_shexp + (size_t)(t - n_dense) * Q8ROW;
        st.fetch_at([&](uint32_t i) {
            const uint32_t c = min(i, NPIECE - 1);
            return c < NPIECE / 2 ? g + 16 * c : u + 16 * (c - NPIECE / 2);
        }, lane);
    }

    float scale = 1.f;
    const float* xrow = x;
    if constexpr (MODE != 0) {
        __shared__ __attribute__((aligned(16))) float s_x[256 * NCH];
        __shared__ float s_red[ROUTE_WAVES];
        scale = stage_normed_row<64 * ROUTE_WAVES, 64 * NCH, MODE == 2>(x, na.w, na.eps, s_x, s_red, aa, blockIdx.x == 0);
        xrow = s_x;
    }

    if (dense) {
        const float4* xv = (const float4*)xrow;
        float4 xx[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) xx[i] = xv[lane + 64 * i];
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            a0 += w[i].x * xx[i].x + w[i].y * xx[i].y;
            a1 += w[i].z * xx[i].z + w[i].w * xx[i].w;
        }
        const float s = wave_sum(a0 + a1) * scale;
        if (lane == 0) ws.logits[t] = s;
    } else if (shared) {
        XSlice xs[P];
#pragma unroll
        for (int p = 0; p < P; p++) load_xslice<QKK_Q8_0>(xs[p], xrow + p * 2048, lane);
        uint8_t* area = s_stage[wave];
        st.commit(area, lane);
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int p = 0; p < P; p++) {
            LaneW<QKK_Q8_0> wg, wu;
            lane_load_lds<QKK_Q8_0>(wg, area, p * 64 * Q8_0_BYTES, lane);
            lane_load_lds<QKK_Q8_0>(wu, area, Q8ROW + p * 64 * Q8_0_BYTES, lane);
            g += wg.dot(xs[p], nullptr, nullptr, lane);
            u += wu.dot(xs[p], nullptr, nullptr, lane);
        }
        g = wave_sum(g) * scale;
        u = wave_sum(u) * scale;
        if (lane == 0) ws.h[(size_t)d.k * d.F + (t - n_dense)] = (g / (1.f + expf(-g))) * u;
    }
}

// ---- launch 2: select + routed gate/up + SiLU --------------------------------------------
// Every workgroup picks the top-n_used experts itself from the E logits of launch 1 (one wave)
// instead of waiting for a selector launch: the logits, the activation slice and the codebook are
// fetched in one round trip, the picked rows in a second.  Workgroup 0 also writes the router
// record.  Wave task = (pick s, RPW consecutive FFN rows): the gate rows are one contiguous range of
// the expert, the up rows another; both are requested as 16-byte pieces right after the selection
// and go through the wave's LDS area one after the other.  IQ3_XXS rows of H = 2048*PASSES weights;
// the product runs on packed halves (two LDS lookups and two XORs per four weights, v_dot2_f32_f16
// against the activations split into hi + lo halves).  NORM: the RMS norm in front, as in launch 1.
// RANKED: the selection by all four waves with select_block (ranks by counting) instead of select_wave's
// rounds on wave 0.
template <int PASSES, int RPW, bool ROWS, bool NORM, bool RANKED>
__global__ __launch_bounds__(256) void moe_gateup_kernel(const uint8_t* __restrict__ gate_exps,
                                                         const uint8_t* __restrict__ up_exps,
                                                         const float* __restrict__ x, MoeWs ws,
                                                         qkk_sel* __restrict__ sel, MoeDims d, NormArg<NORM> na)
{
    if constexpr (ROWS) { // blockIdx.y = activation row, as in launch 1
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
        sel += blockIdx.y;
    }
    constexpr uint32_t RB = 8 * PASSES * IQ3_XXS_BYTES; // bytes of a row
    constexpr uint32_t NPIECE = RPW * RB / 16;
    constexpr int NP = (NPIECE + 63) / 64;
    static_assert((RPW * RB) % 16 == 0, "a wave's rows must be whole 16-byte pieces");
    __shared__ Iq3HalfTables tab;
    __shared__ float s_log[QKK_MAX_EXPERTS + 8];
    __shared__ qkk_sel s_sel;
    __shared__ __attribute__((aligned(16))) uint8_t s_stage[4][WaveStage<NP>::AREA + 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    // round trip 1: codebook word, logits (wave 0), activation slice
    const uint32_t grid_word = g_iq3xxs_grid[threadIdx.x];
    float lv[QKK_MAX_EXPERTS / 64 + 1];
    float l0 = 0.f, l1 = 0.f, lsh = 0.f;
    if constexpr (RANKED) { // thread t: experts t and t + 256; thread 0 also the shared gate's logit
        l0 = threadIdx.x < d.E ? ws.logits[threadIdx.x] : 0.f;
        l1 = threadIdx.x + 256u < d.E ? ws.logits[threadIdx.x + 256u] : 0.f;
        lsh = threadIdx.x == 0 ? ws.logits[d.E] : 0.f;
    } else if (wave == 0) {
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            lv[i] = (uint32_t)(lane + 64 * i) <= d.E ? ws.logits[lane + 64 * i] : 0.f;
    }
    XSliceH xs[PASSES];
    float scale = 1.f;
    if constexpr (NORM) {
        __shared__ __attribute__((aligned(16))) float s_x[2048 * PASSES];
        __shared__ float s_red[4];
        scale = stage_normed_row<256, 512 * PASSES, false>(x, na.w, na.eps, s_x, s_red, AddArg<false>{}, false);
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            XSlice f;
            load_xslice<QKK_IQ3_XXS>(f, s_x + p * 2048, lane);
            split_xslice(xs[p], f);
        }
    } else {
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            XSlice f;
            load_xslice<QKK_IQ3_XXS>(f, x + p * 2048, lane);
            split_xslice(xs[p], f);
        }
    }

    fill_iq3_half_entry(tab, threadIdx.x, grid_word);
    if constexpr (RANKED) {
        __shared__ SelectScratch s_scr;
        select_block(l0, l1, lsh, d.E, d.k, &s_sel, s_scr);
    } else if (wave == 0) {
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            if ((uint32_t)(lane + 64 * i) <= d.E) s_log[lane + 64 * i] = lv[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        select_wave(s_log, d.E, d.k, &s_sel);
        if (lane == 0) s_sel.w_shared = 1.f / (1.f + expf(-s_log[d.E]));
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x < 33) {
        if (threadIdx.x < 16) {
            if (threadIdx.x < d.k) {
                sel->ids[threadIdx.x] = s_sel.ids[threadIdx.x];
                sel->w[threadIdx.x] = s_sel.w[threadIdx.x];
            }
        } else if (threadIdx.x == 32) {
            sel->w_shared = s_sel.w_shared;
        }
    }

    // round trip 2: the picked rows
    const uint32_t groups = d.F / RPW; // row groups per pick (the launcher checks F % RPW == 0)
    uint8_t* area = s_stage[wave];
    for (uint32_t t = blockIdx.x * 4 + wave; t < d.k * groups; t += gridDim.x * 4) {
        const uint32_t s = t / groups, r0 = (t % groups) * RPW;
        const uint32_t e = min(s_sel.ids[s], d.E - 1);
        WaveStage<NP> sg, su;
        sg.fetch(gate_exps + ((size_t)e * d.F + r0) * RB, NPIECE, lane);
        su.fetch(up_exps + ((size_t)e * d.F + r0) * RB, NPIECE, lane);
        float g[RPW], u[RPW];
        sg.commit(area, lane);
#pragma unroll
        for (int i = 0; i < RPW; i++) {
            float a = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                LaneW<QKK_IQ3_XXS> w;
                lane_load_lds<QKK_IQ3_XXS>(w, area, i * RB + p * 8 * IQ3_XXS_BYTES, lane);
                a += w.dot_h(xs[p], &tab);
            }
            g[i] = wave_sum(a) * scale;
        }
        su.commit(area, lane); // LDS operations of a wave run in order: the reads above are done
#pragma unroll
        for (int i = 0; i < RPW; i++) {
            float a = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                LaneW<QKK_IQ3_XXS> w;
                lane_load_lds<QKK_IQ3_XXS>(w, area, i * RB + p * 8 * IQ3_XXS_BYTES, lane);
                a += w.dot_h(xs[p], &tab);
            }
            u[i] = wave_sum(a) * scale;
        }
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < RPW; i++) ws.h[(size_t)s * d.F + r0 + i] = (g[i] / (1.f + expf(-g[i]))) * u[i];
        }
    }
}

// ---- launch 3: routed down + shared down + combine ---------------------------------------
// Wave task = RIF consecutive outputs o.  F = 32*LPR: LPR lanes cover one down row, so 64/LPR picks
// are processed side by side, in ROUNDS rounds; the shared Q8_0 row rides on lane group 0.
// Round trip 1 fetches everything that does not depend on the picks (router record, h, shared rows,
// codebook); round trip 2 the picked experts' rows: for every pick the RIF rows are one contiguous
// run of its expert, fetched as 16-byte pieces (all picks' runs in one set of loads) into the wave's
// LDS area.  Every wave needs all of h: fetched once per workgroup and shared through LDS.
template <bool ON>
struct ResidArg {
    const float* p;
};
template <>
struct ResidArg<false> {};

// LDS of the down launch, carved from one dynamic allocation.
template <int TYPE, int LPR, int ROUNDS, int RIF>
struct DownShape {
    static constexpr int GROUPS = WAVE / LPR, PICKS = ROUNDS * GROUPS;
    static constexpr uint32_t F = 32 * LPR;
    static constexpr uint32_t RB = (uint32_t)qkk_row_bytes_dev<TYPE>(F), RUN = RIF * RB;
    // a run starts at a multiple of RUN bytes inside its expert (whose size is a multiple of 16)
    static constexpr uint32_t NRUN = RUN % 16 == 0 ? RUN / 16 : (RUN + 14 + 15) / 16; // pieces per pick, from the 16-byte boundary below
    static_assert(RUN % 2 == 0 && (TYPE != QKK_IQ4_XS || RUN % 8 == 0), "runs start on 2-byte (IQ4_XS: 8-byte) boundaries");
    static constexpr int NP = (PICKS * NRUN + 63) / 64;
    static constexpr uint32_t Q8ROW = F / 32 * Q8_0_BYTES, SRUN = RIF * Q8ROW;
    static_assert(SRUN % 16 == 0, "shared rows must be whole 16-byte pieces");
    static constexpr int NPS = (SRUN / 16 + 63) / 64;
    static constexpr uint32_t WAVE_LDS = WaveStage<NP>::AREA + WaveStage<NPS>::AREA + 32;
    // whether the IQ4_XS product runs on packed halves (its activation slices take 32 registers per round)
    static constexpr bool HALF = TYPE == QKK_IQ4_XS && ROUNDS <= 2;
    static size_t lds_bytes(uint32_t k) { return (size_t)(k + 1) * F * 4 + 4 * WAVE_LDS; }
};

// RESID: y = resid + step (the residual row may be y: an element is read and written by the same lane).
template <int TYPE, int LPR, int ROUNDS, int RIF, bool RESID, bool ROWS>
__global__ __launch_bounds__(256) void moe_down_kernel(const uint8_t* __restrict__ down_exps,
                                                       const uint8_t* __restrict__ down_shexp,
                                                       MoeWs ws, const qkk_sel* __restrict__ sel,
                                                       float* y, MoeDims d, ResidArg<RESID> ra)
{
    using S = DownShape<TYPE, LPR, ROUNDS, RIF>;
    if constexpr (ROWS) { // blockIdx.y = activation row, as in launch 1
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
        sel += blockIdx.y;
        y += (size_t)blockIdx.y * d.H;
        if constexpr (RESID) ra.p += (size_t)blockIdx.y * d.H;
    }
    QK_DYN_LDS(uint8_t, s_dyn);
    float* s_h = (float*)s_dyn; // [(k+1)][F]: the gated activations of every pick
    __shared__ IqTables tab;
    __shared__ Iq4PairTable tab4;
    __shared__ uint32_t s_eid[QKK_MAX_USED];
    __shared__ float s_wt[QKK_MAX_USED + 1];
    constexpr int GROUPS = S::GROUPS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    uint8_t* area = s_dyn + (size_t)(d.k + 1) * d.F * 4 + (size_t)wave * S::WAVE_LDS;
    uint8_t* sarea = area + WaveStage<S::NP>::AREA + 16;
    const uint32_t o0 = min((blockIdx.x * 4 + wave) * RIF, d.H - RIF); // the grid covers every output once (H % RIF == 0)
    const bool live = (blockIdx.x * 4 + wave) * RIF < d.H;

    // round trip 1: everything that does not depend on the picks
    uint32_t my_eid = 0;
    float my_wt = 0.f;
    if (threadIdx.x < QKK_MAX_USED) {
        const uint32_t sc = threadIdx.x < d.k ? threadIdx.x : 0;
        my_eid = sel->ids[sc];
        my_wt = threadIdx.x < d.k ? sel->w[sc] : 0.f;
    } else if (threadIdx.x == QKK_MAX_USED) {
        my_wt = sel->w_shared;
    }
    float res[RIF];
#pragma unroll
    for (int i = 0; i < RIF; i++) {
        if constexpr (RESID) res[i] = ra.p[o0 + i];
        else res[i] = 0.f;
    }
    const uint32_t h_quads = (d.k + 1) * d.F / 4;
    constexpr int HQ = 8; // quads per thread in flight: covers (16 + 1) * 1024 / 4 / 256 = 17 in three rounds
    const float4* hg = (const float4*)ws.h;
    float4 hq[HQ];
#pragma unroll
    for (int i = 0; i < HQ; i++) hq[i] = hg[min(threadIdx.x + 256u * i, h_quads - 1)];
    WaveStage<S::NPS> ss;
    ss.fetch(down_shexp + (size_t)o0 * S::Q8ROW, S::SRUN / 16, lane);
    if constexpr (S::HALF) fill_iq4_pair_entry(tab4, threadIdx.x);
    else fill_iq_tables(tab, g_iq3xxs_grid, threadIdx.x, 256);
#pragma unroll
    for (int i = 0; i < HQ; i++) // keeps the loads of h above this line, all in flight at once: sunk into the guarded stores below, they ran one after the other
        asm volatile("" : QK_REG(hq[i].x), QK_REG(hq[i].y), QK_REG(hq[i].z), QK_REG(hq[i].w));
    if (threadIdx.x < QKK_MAX_USED) s_eid[threadIdx.x] = min(my_eid, d.E - 1);
    if (threadIdx.x <= QKK_MAX_USED) s_wt[threadIdx.x] = my_wt;
#pragma unroll
    for (int i = 0; i < HQ; i++)
        if (threadIdx.x + 256u * i < h_quads) ((float4*)s_h)[threadIdx.x + 256u * i] = hq[i];
    for (uint32_t q4 = threadIdx.x + 256u * HQ; q4 < h_quads; q4 += 256u) ((float4*)s_h)[q4] = hg[q4]; // wide layers only
    ss.commit(sarea, lane);
    __syncthreads(); // the picks, h and the codebook in LDS

    // round trip 2: the picks' runs
    const uint32_t A = ((size_t)o0 * S::RB) & 15u; // where a run starts behind its 16-byte boundary
    WaveStage<S::NP> st;
    {
        const uint8_t* base = down_exps + (size_t)o0 * S::RB - A;
        const size_t expert_bytes = (size_t)d.H * S::RB;
        // NRUN is the largest piece count over the possible start offsets A; pieces behind the run's
        // last byte are not needed and may lie behind the end of the tensor: re-read the last one
        const uint32_t last = (A + S::RUN - 1) / 16;
        st.fetch_at([&](uint32_t i) {
            const uint32_t c = min(i, (uint32_t)(S::PICKS * S::NRUN) - 1), pick = c / S::NRUN, idx = min(c % S::NRUN, last);
            return base + (size_t)s_eid[min(pick, d.k - 1)] * expert_bytes + 16 * idx;
        }, lane);
    }
    // while they travel: this lane's slices of h and its weights
    float wt[ROUNDS];
#pragma unroll
    for (int q = 0; q < ROUNDS; q++) {
        const uint32_t s = q * GROUPS + grp;
        wt[q] = s < d.k ? s_wt[s] : 0.f;
    }
    const float wsh = grp == 0 ? s_wt[QKK_MAX_USED] : 0.f;
    XSlice hsh;
    load_xslice<QKK_Q8_0>(hsh, s_h + (size_t)d.k * d.F, lir);
    float shared_part[RIF];
#pragma unroll
    for (int i = 0; i < RIF; i++) {
        LaneW<QKK_Q8_0> wq;
        lane_load_lds<QKK_Q8_0>(wq, sarea, i * S::Q8ROW, lir);
        shared_part[i] = wsh * wq.dot(hsh, nullptr, nullptr, lir);
    }
    float acc[RIF];
    if constexpr (S::HALF) {
        XSliceH hs[ROUNDS];
#pragma unroll
        for (int q = 0; q < ROUNDS; q++) {
            const uint32_t s = q * GROUPS + grp;
            XSlice f;
            load_xslice<TYPE>(f, s_h + (size_t)(s < d.k ? s : 0) * d.F, lir);
            split_xslice_iq4(hs[q], f);
        }
        st.commit(area, lane);
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            acc[i] = shared_part[i];
#pragma unroll
            for (int q = 0; q < ROUNDS; q++) {
                LaneW<TYPE> w;
                lane_load_lds<TYPE>(w, area, (q * GROUPS + grp) * S::NRUN * 16 + A + i * S::RB, lir);
                acc[i] += wt[q] * w.dot_h(hs[q], &tab4, lir);
            }
        }
    } else {
        XSlice hs[ROUNDS];
        float hsum[ROUNDS][4];
#pragma unroll
        for (int q = 0; q < ROUNDS; q++) {
            const uint32_t s = q * GROUPS + grp;
            load_xslice<TYPE>(hs[q], s_h + (size_t)(s < d.k ? s : 0) * d.F, lir);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                float a = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) a += hs[q].v[c * 8 + i];
                hsum[q][c] = a;
            }
        }
        st.commit(area, lane);
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            acc[i] = shared_part[i];
#pragma unroll
            for (int q = 0; q < ROUNDS; q++) {
                LaneW<TYPE> w;
                lane_load_lds<TYPE>(w, area, (q * GROUPS + grp) * S::NRUN * 16 + A + i * S::RB, lir);
                acc[i] += wt[q] * w.dot(hs[q], hsum[q], &tab, lir);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RIF; i++) {
        float a = wave_sum(acc[i]);
        if constexpr (RESID) a += res[i];
        if (lane == 0 && live) y[o0 + i] = a;
    }
}

} // namespace qk

namespace qk {
int moe_grouped_launch(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                       uint32_t N, uint32_t stages, hipStream_t st, const MoeTail* tail);
int moe_ws_alarm_take(bool* was_set);
void launch_add_rmsnorm(const float* a, const float* b, const float* w, float* y, float* xn, uint32_t n, uint32_t rows,
                        float eps, hipStream_t st);
}
using namespace qk;

static int check_layer(const qkk_moe_layer* L, const char* who)
{
    if (!L) return fail(QKK_EINVAL, "%s: null layer", who);
    if (!L->gate_inp || !L->gate_inp_shexp || !L->gate_exps || !L->up_exps || !L->down_exps ||
        !L->gate_shexp || !L->up_shexp || !L->down_shexp)
        return fail(QKK_EINVAL, "%s: null tensor pointer", who);
    if (L->gu_type != QKK_IQ3_XXS) return fail(QKK_ETYPE, "%s: gate/up experts must be IQ3_XXS", who);
    if (L->down_type != QKK_IQ4_XS && L->down_type != QKK_Q6_K)
        return fail(QKK_ETYPE, "%s: down experts must be IQ4_XS or Q6_K", who);
    if (L->n_embd != 2048 && L->n_embd != 4096)
        return fail(QKK_ESHAPE, "%s: n_embd %u not supported (2048 or 4096)", who, L->n_embd);
    if ((L->n_ff != 512 && L->n_ff != 256 && L->n_ff != 1024) || (L->n_ff == 1024 && L->n_used > 16))
        return fail(QKK_ESHAPE, "%s: n_ff %u not supported (256, 512 or 1024)", who, L->n_ff);
    if (L->n_expert < 1 || L->n_expert > QKK_MAX_EXPERTS)
        return fail(QKK_ESHAPE, "%s: n_expert %u outside 1..%u", who, L->n_expert, QKK_MAX_EXPERTS);
    if (L->n_used < 1 || L->n_used > QKK_MAX_USED || L->n_used > L->n_expert)
        return fail(QKK_ESHAPE, "%s: n_used %u outside 1..min(16, n_expert)", who, L->n_used);
    const void* t[] = {L->gate_inp, L->gate_inp_shexp, L->gate_exps, L->up_exps,
                       L->down_exps, L->gate_shexp, L->up_shexp, L->down_shexp};
    for (const void* p : t)
        if (!aligned16(p)) return fail(QKK_EINVAL, "%s: tensors must be 16-byte aligned", who);
    return QKK_OK;
}

template <int TYPE, int LPR, int ROUNDS, int RIF>
static void launch_down2(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y,
                         const MoeDims& d, const float* resid, uint32_t rows, hipStream_t st)
{
    using S = DownShape<TYPE, LPR, ROUNDS, RIF>;
    const uint32_t waves = (d.H + RIF - 1) / RIF;
    const uint32_t lds = (uint32_t)S::lds_bytes(d.k); // h [(k+1)][F] + the waves' staging areas
    static bool raised = [] {
        const int most = (int)S::lds_bytes(QKK_MAX_USED);
        for (const void* f : {(const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, false>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, false>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, true>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, true>})
            (void)hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, most);
        return true;
    }();
    (void)raised;
    const dim3 grid((waves + 3) / 4, rows), block(256);
    const uint8_t *de = (const uint8_t*)L->down_exps, *ds = (const uint8_t*)L->down_shexp;
    if (rows > 1 && resid)
        hipLaunchKernelGGL((moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, true>), grid, block, lds, st, de, ds, ws, sel, Y,
                           d, ResidArg<true>{resid});
    else if (rows > 1)
        hipLaunchKernelGGL((moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, true>), grid, block, lds, st, de, ds, ws, sel, Y,
                           d, ResidArg<false>{});
    else if (resid)
        hipLaunchKernelGGL((moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, false>), grid, block, lds, st, de, ds, ws, sel, Y,
                           d, ResidArg<true>{resid});
    else
        hipLaunchKernelGGL((moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, false>), grid, block, lds, st, de, ds, ws, sel, Y,
                           d, ResidArg<false>{});
}

// Picks processed side by side = 64/LPR; ROUNDS covers n_used with the fewest passes and
// the rows in flight shrink as ROUNDS grows so the lane's registers hold them.  With eight picks
// two outputs per wave (one workgroup per CU at n_embd = 2048) measured 7.7 us against 9.9 us for
// four outputs per wave, which leaves half the CUs without work.
template <int TYPE, int LPR>
static void launch_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y,
                        const MoeDims& d, const float* resid, uint32_t rows, hipStream_t st)
{
    const uint32_t need = (d.k + 64 / LPR - 1) / (64 / LPR);
    if (need <= 1) launch_down2<TYPE, LPR, 1, 4>(L, ws, sel, Y, d, resid, rows, st);
    else if (need <= 2) launch_down2<TYPE, LPR, 2, 2>(L, ws, sel, Y, d, resid, rows, st); // 256 workgroups at n_embd 2048
    else if (need <= 4) launch_down2<TYPE, LPR, 4, 2>(L, ws, sel, Y, d, resid, rows, st);
    else launch_down2<TYPE, LPR, 8, 1>(L, ws, sel, Y, d, resid, rows, st);
}

template <int TYPE>
static void launch_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y,
                        const MoeDims& d, const float* resid, uint32_t rows, hipStream_t st)
{
    if (d.F == 512) launch_down<TYPE, 16>(L, ws, sel, Y, d, resid, rows, st);
    else if (d.F == 256) launch_down<TYPE, 8>(L, ws, sel, Y, d, resid, rows, st);
    else launch_down<TYPE, 32>(L, ws, sel, Y, d, resid, rows, st);
}

constexpr uint32_t ROWWISE_MAX = QKK_ROWWISE_MAX; // rows up to which each row runs the one-row launches

// Launches 1 and 2 for `rows` activation rows (grid.y); norm given: the variants with the RMS norm
// in front.
static void launch_route_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, qkk_sel* sel, const MoeDims& d,
                                uint32_t stages, const MoeNorm* norm, uint32_t rows, hipStream_t st)
{
    const uint8_t *gs = (const uint8_t*)L->gate_shexp, *us = (const uint8_t*)L->up_shexp;
    const uint8_t *ge = (const uint8_t*)L->gate_exps, *ue = (const uint8_t*)L->up_exps;
    const bool wide = d.H != 2048; // n_embd 4096
    if (stages & QKK_STAGE_ROUTE) {
        const dim3 grid((d.E + 1 + d.F + ROUTE_WAVES - 1) / ROUTE_WAVES, rows), block(64 * ROUTE_WAVES);
#define QK_ROUTE(NCH, ROWS) \
    do { \
        if (norm && norm->mix) \
            hipLaunchKernelGGL((moe_route_kernel<NCH, ROWS, 2>), grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, \
                               ws, d, NormArg<true>{norm->w, norm->eps}, AddArg<true>{norm->mix, norm->sum}); \
        else if (norm) \
            hipLaunchKernelGGL((moe_route_kernel<NCH, ROWS, 1>), grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, \
                               ws, d, NormArg<true>{norm->w, norm->eps}, AddArg<false>{}); \
        else \
            hipLaunchKernelGGL((moe_route_kernel<NCH, ROWS, 0>), grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, \
                               ws, d, NormArg<false>{}, AddArg<false>{}); \
    } while (0)
        if (!wide && rows > 1) QK_ROUTE(8, true);
        else if (!wide) QK_ROUTE(8, false);
        else if (rows > 1) QK_ROUTE(16, true);
        else QK_ROUTE(16, false);
#undef QK_ROUTE
    }
    if (norm && norm->mix) X = norm->sum; // launch 2 reads the sum launch 1 stored
    if (stages & QKK_STAGE_GATEUP) {
        // FFN rows per wave: four at n_embd 2048, two at 4096 (the same bytes); n_ff is a multiple of both
        const uint32_t rpw = wide ? 2 : 4;
        const dim3 grid((d.k * (d.F / rpw) + 3) / 4, rows), block(256);
        const bool ranked = options().select_ranked != 0; // the selection by rank counting on all four waves
#define QK_GATEUP2(PASSES, RPW, ROWS, RANKED) \
    do { \
        if (norm) \
            hipLaunchKernelGGL((moe_gateup_kernel<PASSES, RPW, ROWS, true, RANKED>), grid, block, 0, st, ge, ue, X, ws, sel, d, \
                               NormArg<true>{norm->w, norm->eps}); \
        else \
            hipLaunchKernelGGL((moe_gateup_kernel<PASSES, RPW, ROWS, false, RANKED>), grid, block, 0, st, ge, ue, X, ws, sel, d, \
                               NormArg<false>{}); \
    } while (0)
#define QK_GATEUP(PASSES, RPW, ROWS) \
    do { \
        if (ranked) QK_GATEUP2(PASSES, RPW, ROWS, true); \
        else QK_GATEUP2(PASSES, RPW, ROWS, false); \
    } while (0)
        if (!wide && rows > 1) QK_GATEUP(1, 4, true);
        else if (!wide) QK_GATEUP(1, 4, false);
        else if (rows > 1) QK_GATEUP(2, 2, true);
        else QK_GATEUP(2, 2, false);
#undef QK_GATEUP
#undef QK_GATEUP2
    }
}

// ---- the step for callers that cannot allocate ---------------------------------------------------
// The workspace of qkk_moe_decode as a file-scope device array: each device the library runs on holds
// its own copy, at its own address, until the process ends.  In host code the array's name is only a
// stand-in for that address; it is resolved once per device (with that device current) and every
// launch takes the resolved pointer.
static __device__ __align__(256) unsigned char scratch[QKK_MOE_STATIC_BYTES];

namespace qk {
constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES]; // resolved device address of `scratch`, per device
static std::mutex g_scratch_mu;

// Address of the current device's copy of the array, or nullptr with the error recorded.
void* moe_static_scratch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        (void)hipGetLastError();
        fail(QKK_EDEVICE, "qkk_moe_decode_static: no current HIP device below %d", MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            fail(QKK_EDEVICE, "qkk_moe_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

// Clears the arrival counters at the head of the workspace (a fill kernel, not a memset node: the
// caller may be capturing a graph).
__global__ void moe_static_clear_kernel(uint32_t* counters)
{
    counters[threadIdx.x] = 0u;
}
} // namespace qk

extern "C" {

size_t qkk_moe_workspace_bytes(const qkk_moe_layer* L, uint32_t n_slots)
{
    if (!L || n_slots == 0) return 0;
    const MoeDims d{L->n_embd, L->n_ff, L->n_expert, L->n_used};
    return ws_bytes(d, n_slots);
}

static int moe_decode_impl(const char* who, const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel,
                           void* workspace, size_t workspace_bytes, uint32_t n_slots, uint32_t stages,
                           void* stream, const MoeTail* tail = nullptr, const MoeNorm* norm = nullptr)
{
    if (int rc = check_layer(L, who)) return rc;
    if (!X || !Y || !sel || !workspace) return fail(QKK_EINVAL, "%s: null pointer", who);
    if (n_slots < 1 || n_slots > 4096) return fail(QKK_ESHAPE, "%s: %u rows outside 1..4096", who, n_slots);
    if (!aligned16(X) || !aligned16(Y) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return fail(QKK_EINVAL, "%s: X/Y must be 16-byte and workspace 256-byte aligned", who);
    const MoeDims d{L->n_embd, L->n_ff, L->n_expert, L->n_used};
    if (workspace_bytes < ws_bytes(d, n_slots))
        return fail(QKK_EWORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes, ws_bytes(d, n_slots));
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    // A few rows hardly ever pick the same expert (4 rows: 30.6 distinct of 32 picks on average), so
    // there is little to share: each row runs the one-row launches (grid.y = row), and its result
    // is bit for bit what it is alone.  Measured: 2 rows 26 us against 40 us on the expert-major
    // path, 4 rows 37 / 50, 8 rows 62 / 71, 10 rows 76 / 78, 12 rows 87 / 86: more rows go there.
    // the "rowwise_max" switch moves the change between the two paths for the plain step, for measurements on
    // the device (the limit of the entry points with the norm in front stays QKK_ROWWISE_MAX)
    const uint32_t switch_opt = (uint32_t)options().rowwise_max;
    if (n_slots > (norm || !switch_opt ? ROWWISE_MAX : switch_opt)) {
        if (norm) return fail(QKK_ESHAPE, "%s: %u rows exceed %u (use qkk_moe_decode_tail)", who, n_slots, ROWWISE_MAX);
        return moe_grouped_launch(L, X, Y, sel, workspace, n_slots, stages, st, tail);
    }
    const MoeWs ws = ws_carve(workspace, d, n_slots);

    // two forms of the three launches: block fields loaded per lane (qk_moe_lane.hip), or rows streamed
    // as 16-byte pieces through LDS (this file); same arguments, same workspace
    const bool staged = options().one_row_stream != 0;
    if (staged) launch_route_gateup(L, X, ws, sel, d, stages, norm, n_slots, st);
    else lane_route_gateup(L, X, ws, sel, d, stages, norm, n_slots, st);
    if (stages & QKK_STAGE_DOWN) {
        // norm in front: the input row (with the mixer's output, if any) is the residual; Y may be X
        const float* resid = norm ? (norm->mix ? norm->sum : X) : nullptr;
        if (!staged) lane_down(L, ws, sel, Y, d, resid, n_slots, st);
        else if (L->down_type == QKK_IQ4_XS) launch_down<QKK_IQ4_XS>(L, ws, sel, Y, d, resid, n_slots, st);
        else launch_down<QKK_Q6_K>(L, ws, sel, Y, d, resid, n_slots, st);
        // the step's output went to tail->Xn (see qkk_moe_decode_tail); add and norm in place
        if (tail) launch_add_rmsnorm(tail->resid, Y, tail->w_next, tail->S, tail->Xn, d.H, n_slots, tail->eps, st);
    }
    return check_launch(who);
}

int qkk_moe_decode(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                   size_t workspace_bytes, uint32_t n_slots, void* stream)
{
    return moe_decode_impl("qkk_moe_decode", L, X, Y, sel, workspace, workspace_bytes, n_slots, QKK_STAGE_ALL,
                           stream);
}

int qkk_moe_workspace_status(void* stream)
{
    if (int rc = require_device()) return rc;
    if (hipStreamSynchronize(as_stream(stream)) != hipSuccess) {
        (void)hipGetLastError();
        return fail(QKK_EDEVICE, "qkk_moe_workspace_status: the stream failed");
    }
    bool dirty = false;
    if (int rc = moe_ws_alarm_take(&dirty)) return rc;
    if (dirty)
        return fail(QKK_EINVAL, "qkk_moe_workspace_status: a call with more than %u rows ran on a workspace whose header "
                    "was not zero (never cleared, or the clear had not completed): its results are invalid", ROWWISE_MAX);
    return QKK_OK;
}

int qkk_moe_decode_static(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, uint32_t n_slots,
                          void* stream)
{
    const char* who = "qkk_moe_decode_static";
    if (int rc = check_layer(L, who)) return rc;
    if (n_slots < 1 || n_slots > QKK_MOE_STATIC_MAX_SLOTS)
        return fail(QKK_ESHAPE, "%s: %u rows outside 1..%u", who, n_slots, QKK_MOE_STATIC_MAX_SLOTS);
    const MoeDims d{L->n_embd, L->n_ff, L->n_expert, L->n_used};
    if (ws_bytes(d, n_slots) > QKK_MOE_STATIC_BYTES)
        return fail(QKK_EWORKSPACE, "%s: this layer shape with %u rows needs %zu bytes of workspace, the static array holds %u",
                    who, n_slots, ws_bytes(d, n_slots), QKK_MOE_STATIC_BYTES);
    if (int rc = require_device()) return rc;
    void* ws = moe_static_scratch();
    if (!ws) return QKK_EDEVICE;
    // The array keeps what the last call left.  Logits, h, pair lists and contributions are written
    // before they are read; the arrival counters of the expert-major path must start at zero.
    if (n_slots > ROWWISE_MAX)
        hipLaunchKernelGGL(moe_static_clear_kernel, dim3(1), dim3(64), 0, as_stream(stream), (uint32_t*)ws);
    return moe_decode_impl(who, L, X, Y, sel, ws, QKK_MOE_STATIC_BYTES, n_slots, QKK_STAGE_ALL, stream);
}

int qkk_moe_decode_tail(const qkk_moe_layer* L, const float* X, const float* resid, const float* w_next, float eps,
                        float* S, float* Xn, qkk_sel* sel, void* workspace, size_t workspace_bytes, uint32_t n_slots,
                        void* stream)
{
    if (!resid || !w_next || !S || !Xn) return fail(QKK_EINVAL, "qkk_moe_decode_tail: null pointer");
    if (!aligned16(resid) || !aligned16(w_next) || !aligned16(S) || !aligned16(Xn))
        return fail(QKK_EINVAL, "qkk_moe_decode_tail: resid, w_next, S and Xn must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_moe_decode_tail: eps must be non-negative");
    if (Xn == X || Xn == resid || Xn == S)
        return fail(QKK_EINVAL, "qkk_moe_decode_tail: Xn must be a buffer of its own (it holds the step's output on the way)");
    const MoeTail tail{resid, w_next, eps, S, Xn};
    // the step writes its output row(s) to Xn when it has to materialise them (one row)
    return moe_decode_impl("qkk_moe_decode_tail", L, X, Xn, sel, workspace, workspace_bytes, n_slots, QKK_STAGE_ALL, stream,
                           &tail);
}

int qkk_moe_layer_rows(const qkk_moe_layer* L, float* S, const float* w_norm, float eps, qkk_sel* sel, void* workspace,
                       size_t workspace_bytes, uint32_t n_slots, void* stream)
{
    if (!w_norm) return fail(QKK_EINVAL, "qkk_moe_layer_rows: null pointer");
    if (!aligned16(w_norm)) return fail(QKK_EINVAL, "qkk_moe_layer_rows: w_norm must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_moe_layer_rows: eps must be non-negative");
    const MoeNorm norm{w_norm, eps};
    return moe_decode_impl("qkk_moe_layer_rows", L, S, S, sel, workspace, workspace_bytes, n_slots, QKK_STAGE_ALL, stream,
                           nullptr, &norm);
}

int qkk_moe_layer_rows_add(const qkk_moe_layer* L, float* S, const float* mix, float* T, const float* w_norm, float eps,
                           qkk_sel* sel, void* workspace, size_t workspace_bytes, uint32_t n_slots, void* stream)
{
    if (!w_norm || !mix || !T) return fail(QKK_EINVAL, "qkk_moe_layer_rows_add: null pointer");
    if (!aligned16(w_norm) || !aligned16(mix) || !aligned16(T))
        return fail(QKK_EINVAL, "qkk_moe_layer_rows_add: w_norm, mix and T must be 16-byte aligned");
    if (T == S || T == mix) return fail(QKK_EINVAL, "qkk_moe_layer_rows_add: T must be a buffer of its own");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_moe_layer_rows_add: eps must be non-negative");
    const MoeNorm norm{w_norm, eps, mix, T};
    return moe_decode_impl("qkk_moe_layer_rows_add", L, S, S, sel, workspace, workspace_bytes, n_slots, QKK_STAGE_ALL,
                           stream, nullptr, &norm);
}

int qkk_moe_decode_stages(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                          size_t workspace_bytes, uint32_t n_slots, uint32_t stages, void* stream)
{
    if ((stages & ~QKK_STAGE_ALL) || stages == 0)
        return fail(QKK_EINVAL, "qkk_moe_decode_stages: stage mask 0x%x outside 1..7", stages);
    return moe_decode_impl("qkk_moe_decode_stages", L, X, Y, sel, workspace, workspace_bytes, n_slots, stages,
                           stream);
}

} // extern "C"
