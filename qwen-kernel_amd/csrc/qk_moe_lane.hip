// qk_moe_lane.hip -- the one-row fused MoE step with per-lane block loads.
//
// The three launches of qk_moe.hip (route, select + gate/up, down + combine) in the form in which
// every lane fetches its own block fields from global memory (LaneW<TYPE>::load).  This is the form
// whose results and timings come from runs on an MI355X; the step uses it unless the "one_row" switch
// selects the streaming kernels of qk_moe.hip.  On this device a dependent memory access costs 2-3 us
// when the line is cold while a kernel boundary costs well under 1 us, so each launch is arranged as
// two round trips at most and nothing synchronises inside a kernel.
#include "qk_moe_common.h"

namespace qk {
namespace lane {

// ---- launch 1: router logits + shared gate/up ---------------------------------------------
// One wave per task, no loop: tasks [0, E] are F32 rows (row E = the shared gate row), tasks
// after that are shared-expert gate/up row pairs.  Every load of a task is issued before its
// arithmetic, so a task costs one memory round trip.  H = 256*NCH.
// ROWS: blockIdx.y is the activation row (slot); every row runs the one-row launch on its own part
// of x and of the workspace -- for a few rows, which hardly ever pick the same expert, this beats
// the expert-major path, and a row's result does not depend on its company.
template <int NCH, bool ROWS>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ gate_inp,
                                                        const float* __restrict__ gate_inp_shexp,
                                                        const uint8_t* __restrict__ gate_shexp,
                                                        const uint8_t* __restrict__ up_shexp,
                                                        const float* __restrict__ x, MoeWs ws, MoeDims d)
{
    if constexpr (ROWS) {
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
    }
    constexpr int P = NCH / 8; // 2048-weight passes per Q8_0 row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_dense = d.E + 1, n_tasks = n_dense + d.F;
    const uint32_t q8_row = d.H / 32 * Q8_0_BYTES;
    const uint32_t t = blockIdx.x * 4 + wave;

    if (t < n_dense) {
        const float4* row = (const float4*)(t < d.E ? gate_inp + (size_t)t * d.H : gate_inp_shexp);
        const float4* xv = (const float4*)x;
        float4 w[NCH], xx[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
#pragma unroll
        for (int i = 0; i < NCH; i++) xx[i] = xv[lane + 64 * i];
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            a0 += w[i].x * xx[i].x + w[i].y * xx[i].y;
            a1 += w[i].z * xx[i].z + w[i].w * xx[i].w;
        }
        const float s = wave_sum(a0 + a1);
        if (lane == 0) ws.logits[t] = s;
    } else if (t < n_tasks) {
        const uint32_t r = t - n_dense;
        LaneW<QKK_Q8_0> wg[P], wu[P];
        XSlice xs[P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            wg[p].load(gate_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
            wu[p].load(up_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
        }
#pragma unroll
        for (int p = 0; p < P; p++) load_xslice<QKK_Q8_0>(xs[p], x + p * 2048, lane);
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int p = 0; p < P; p++) {
            g += wg[p].dot(xs[p], nullptr, nullptr, lane);
            u += wu[p].dot(xs[p], nullptr, nullptr, lane);
        }
        g = wave_sum(g);
        u = wave_sum(u);
        if (lane == 0) ws.h[(size_t)d.k * d.F + r] = (g / (1.f + expf(-g))) * u;
    }
}

// The same launch with the RMS norm in front: x is the un-normalised residual row; the workgroup
// forms x * nw once, in LDS, and sums the squares (a wave that fetched x and nw for itself made the
// launch 1.7 us longer: three 8 KB rows per wave through the L1 instead of two); the dot products
// run on x * nw and their sums are scaled by 1/sqrt(mean(x^2) + eps), which is common to a row's
// terms.  The task's weights are requested first, so they are in flight while x arrives.
// ADD: the row is x + mix (a mixer's output on top of the residual); the first workgroup of the row
// also stores the sum to `sum`, a buffer of its own, for the launches behind this one.
template <bool ON>
struct AddArg {
    const float* mix;
    float* sum;
};
template <>
struct AddArg<false> {};

template <int NCH, bool ROWS, bool ADD = false>
__global__ __launch_bounds__(256) void moe_route_norm_kernel(const float* __restrict__ gate_inp,
                                                        const float* __restrict__ gate_inp_shexp,
                                                        const uint8_t* __restrict__ gate_shexp,
                                                        const uint8_t* __restrict__ up_shexp,
                                                        const float* __restrict__ x, MoeWs ws, MoeDims d,
                                                        const float* __restrict__ nw, float eps, AddArg<ADD> aa)
{
    if constexpr (ROWS && ADD) {
        aa.mix += (size_t)blockIdx.y * d.H;
        aa.sum += (size_t)blockIdx.y * d.H;
    }
    if constexpr (ROWS) {
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
    }
    constexpr int P = NCH / 8; // 2048-weight passes per Q8_0 row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_dense = d.E + 1, n_tasks = n_dense + d.F;
    const uint32_t q8_row = d.H / 32 * Q8_0_BYTES;
    const uint32_t t = blockIdx.x * 4 + wave;

    // the task's weights first: they are in flight while x arrives
    const bool dense = t < n_dense, shared = !dense && t < n_tasks;
    float4 w[NCH];
    LaneW<QKK_Q8_0> wg[P], wu[P];
    if (dense) {
        const float4* row = (const float4*)(t < d.E ? gate_inp + (size_t)t * d.H : gate_inp_shexp);
#pragma unroll
        for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
    } else if (shared) {
        const uint32_t r = t - n_dense;
#pragma unroll
        for (int p = 0; p < P; p++) {
            wg[p].load(gate_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
            wu[p].load(up_shexp + (size_t)r * q8_row + (size_t)p * 64 * Q8_0_BYTES, lane);
        }
    }

    __shared__ __attribute__((aligned(16))) float s_x[256 * NCH];
    __shared__ float s_red[4];
    float scale = 1.f;
    const float* xrow = x;
    {
        float4 xv[NCH / 4], nv[NCH / 4];
#pragma unroll
        for (int i = 0; i < NCH / 4; i++) xv[i] = ((const float4*)x)[threadIdx.x + 256 * i];
#pragma unroll
        for (int i = 0; i < NCH / 4; i++) nv[i] = ((const float4*)nw)[threadIdx.x + 256 * i];
        if constexpr (ADD) {
#pragma unroll
            for (int i = 0; i < NCH / 4; i++) {
                const float4 m = ((const float4*)aa.mix)[threadIdx.x + 256 * i];
                xv[i] = float4{xv[i].x + m.x, xv[i].y + m.y, xv[i].z + m.z, xv[i].w + m.w};
                if (blockIdx.x == 0) ((float4*)aa.sum)[threadIdx.x + 256 * i] = xv[i];
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NCH / 4; i++) {
            ss += (xv[i].x * xv[i].x + xv[i].y * xv[i].y) + (xv[i].z * xv[i].z + xv[i].w * xv[i].w);
            ((float4*)s_x)[threadIdx.x + 256 * i] =
                float4{xv[i].x * nv[i].x, xv[i].y * nv[i].y, xv[i].z * nv[i].z, xv[i].w * nv[i].w};
        }
        scale = 1.f / sqrtf(block_sum4(ss, s_red) / (float)d.H + eps); // its barrier also publishes s_x
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
        const uint32_t r = t - n_dense;
        XSlice xs[P];
#pragma unroll
        for (int p = 0; p < P; p++) load_xslice<QKK_Q8_0>(xs[p], xrow + p * 2048, lane);
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int p = 0; p < P; p++) {
            g += wg[p].dot(xs[p], nullptr, nullptr, lane);
            u += wu[p].dot(xs[p], nullptr, nullptr, lane);
        }
        g = wave_sum(g) * scale;
        u = wave_sum(u) * scale;
        if (lane == 0) ws.h[(size_t)d.k * d.F + r] = (g / (1.f + expf(-g))) * u;
    }
}

// ---- launch 2: select + routed gate/up + SiLU --------------------------------------------
// Every workgroup picks the top-n_used experts itself from the E logits of launch 1 (one wave,
// ~1.7 us) instead of waiting for a selector launch: the logits, the activation slice and the
// codebook are fetched in one round trip, the picked rows in a second.  Workgroup 0 also
// writes the router record.  Wave task = (pick s, RIF consecutive FFN rows); gate and up rows
// of one FFN row are fetched together.  IQ3_XXS rows of H = 2048*PASSES weights.  A workgroup's
// time line, measured with the device clock: round trip 1 about 1.5 us, selection 1.7 us, second
// round trip and first row 1.9 us, the other rows 2.6 us (arrival of the picked experts' 6.4 MB,
// not arithmetic: the product on packed halves -- two LDS lookups and two XORs per four weights,
// v_dot2_f32_f16 against the activations split into hi + lo halves -- cut the launch by 0.2 us).
template <int TYPE, int PASSES, int RIF, bool ROWS>
__global__ __launch_bounds__(256) void moe_gateup_kernel(const uint8_t* __restrict__ gate_exps,
                                                         const uint8_t* __restrict__ up_exps,
                                                         const float* __restrict__ x, MoeWs ws,
                                                         qkk_sel* __restrict__ sel, MoeDims d)
{
    if constexpr (ROWS) { // blockIdx.y = activation row, as in launch 1
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
        sel += blockIdx.y;
    }
    __shared__ Iq3HalfTables tab;
    __shared__ float s_log[QKK_MAX_EXPERTS + 8];
    __shared__ qkk_sel s_sel;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row_bytes = (uint32_t)qkk_row_bytes_dev<TYPE>(d.H);
    const uint32_t pass_bytes = row_bytes / PASSES;

    // round trip 1: codebook word, logits (wave 0), activation slice
    const uint32_t grid_word = g_iq3xxs_grid[threadIdx.x];
    float lv[QKK_MAX_EXPERTS / 64 + 1];
    if (wave == 0) {
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            lv[i] = (uint32_t)(lane + 64 * i) <= d.E ? ws.logits[lane + 64 * i] : 0.f;
    }
    XSliceH xs[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        XSlice f;
        load_xslice<TYPE>(f, x + p * 2048, lane);
        split_xslice(xs[p], f);
    }

    fill_iq3_half_entry(tab, threadIdx.x, grid_word);
    if (wave == 0) {
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

    const uint32_t groups = (d.F + RIF - 1) / RIF; // row groups per pick
    for (uint32_t t = blockIdx.x * 4 + wave; t < d.k * groups; t += gridDim.x * 4) {
        const uint32_t s = t / groups, r0 = (t % groups) * RIF;
        const uint32_t e = min(s_sel.ids[s], d.E - 1);
        const uint8_t* gbase = gate_exps + ((size_t)e * d.F) * row_bytes;
        const uint8_t* ubase = up_exps + ((size_t)e * d.F) * row_bytes;
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
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                g += wg[i][p].dot_h_inline(xs[p], &tab);
                u += wu[i][p].dot_h_inline(xs[p], &tab);
            }
            g = wave_sum(g);
            u = wave_sum(u);
            if (lane == 0 && r0 + i < d.F) ws.h[(size_t)s * d.F + r0 + i] = (g / (1.f + expf(-g))) * u;
        }
    }
}

// Launch 2 with the RMS norm in front, as moe_route_norm_kernel: x * nw through LDS, sums scaled.
template <int TYPE, int PASSES, int RIF, bool ROWS>
__global__ __launch_bounds__(256) void moe_gateup_norm_kernel(const uint8_t* __restrict__ gate_exps,
                                                         const uint8_t* __restrict__ up_exps,
                                                         const float* __restrict__ x, MoeWs ws,
                                                         qkk_sel* __restrict__ sel, MoeDims d,
                                                         const float* __restrict__ nw, float eps)
{
    if constexpr (ROWS) {
        x += (size_t)blockIdx.y * d.H;
        ws.logits += (size_t)blockIdx.y * lstride(d.E);
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
        sel += blockIdx.y;
    }
    __shared__ Iq3HalfTables tab;
    __shared__ float s_log[QKK_MAX_EXPERTS + 8];
    __shared__ qkk_sel s_sel;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row_bytes = (uint32_t)qkk_row_bytes_dev<TYPE>(d.H);
    const uint32_t pass_bytes = row_bytes / PASSES;

    // round trip 1: codebook word, logits (wave 0), activation slice
    const uint32_t grid_word = g_iq3xxs_grid[threadIdx.x];
    float lv[QKK_MAX_EXPERTS / 64 + 1];
    if (wave == 0) {
#pragma unroll
        for (int i = 0; i <= (int)(QKK_MAX_EXPERTS / 64); i++)
            lv[i] = (uint32_t)(lane + 64 * i) <= d.E ? ws.logits[lane + 64 * i] : 0.f;
    }
    XSliceH xs[PASSES];
    __shared__ __attribute__((aligned(16))) float s_x[2048 * PASSES];
    __shared__ float s_red[4];
    float scale = 1.f;
    { // the workgroup forms x * nw once, in LDS, and sums the squares
        float4 xv[2 * PASSES], nv[2 * PASSES];
#pragma unroll
        for (int i = 0; i < 2 * PASSES; i++) xv[i] = ((const float4*)x)[threadIdx.x + 256 * i];
#pragma unroll
        for (int i = 0; i < 2 * PASSES; i++) nv[i] = ((const float4*)nw)[threadIdx.x + 256 * i];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 2 * PASSES; i++) {
            ss += (xv[i].x * xv[i].x + xv[i].y * xv[i].y) + (xv[i].z * xv[i].z + xv[i].w * xv[i].w);
            ((float4*)s_x)[threadIdx.x + 256 * i] =
                float4{xv[i].x * nv[i].x, xv[i].y * nv[i].y, xv[i].z * nv[i].z, xv[i].w * nv[i].w};
        }
        scale = 1.f / sqrtf(block_sum4(ss, s_red) / (float)(2048 * PASSES) + eps); // its barrier publishes s_x
    }
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        XSlice f;
        load_xslice<TYPE>(f, s_x + p * 2048, lane);
        split_xslice(xs[p], f);
    }

    fill_iq3_half_entry(tab, threadIdx.x, grid_word);
    if (wave == 0) {
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

    const uint32_t groups = (d.F + RIF - 1) / RIF; // row groups per pick
    for (uint32_t t = blockIdx.x * 4 + wave; t < d.k * groups; t += gridDim.x * 4) {
        const uint32_t s = t / groups, r0 = (t % groups) * RIF;
        const uint32_t e = min(s_sel.ids[s], d.E - 1);
        const uint8_t* gbase = gate_exps + ((size_t)e * d.F) * row_bytes;
        const uint8_t* ubase = up_exps + ((size_t)e * d.F) * row_bytes;
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
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                g += wg[i][p].dot_h_inline(xs[p], &tab);
                u += wu[i][p].dot_h_inline(xs[p], &tab);
            }
            g = wave_sum(g) * scale;
            u = wave_sum(u) * scale;
            if (lane == 0 && r0 + i < d.F) ws.h[(size_t)s * d.F + r0 + i] = (g / (1.f + expf(-g))) * u;
        }
    }
}

// ---- launch 3: routed down + shared down + combine ---------------------------------------
// Wave task = RIF consecutive outputs o.  F = 32*LPR: LPR lanes cover one down row, so
// 64/LPR picks are processed side by side; the shared Q8_0 row rides on lane group 0.
// Round trip 1 fetches everything that does not depend on the picks (router record, h slices,
// shared rows, codebook); round trip 2 the picked experts' rows.
template <bool ON>
struct ResidArg {
    const float* p;
};
template <>
struct ResidArg<false> {};

// RESID: y = resid + step (the residual row may be y: an element is read and written by the same lane).
template <int TYPE, int LPR, int ROUNDS, int RIF, bool RESID, bool ROWS>
__global__ __launch_bounds__(256) void moe_down_kernel(const uint8_t* __restrict__ down_exps,
                                                       const uint8_t* __restrict__ down_shexp,
                                                       MoeWs ws, const qkk_sel* __restrict__ sel,
                                                       float* y, MoeDims d, ResidArg<RESID> ra)
{
    if constexpr (ROWS) { // blockIdx.y = activation row, as in launch 1
        ws.h += (size_t)blockIdx.y * (d.k + 1) * d.F;
        sel += blockIdx.y;
        y += (size_t)blockIdx.y * d.H;
        if constexpr (RESID) ra.p += (size_t)blockIdx.y * d.H;
    }
    QK_DYN_LDS(float, s_h); // [(k+1)][F]: the gated activations of every pick
    __shared__ IqTables tab;
    constexpr int GROUPS = WAVE / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const uint32_t row_bytes = (uint32_t)qkk_row_bytes_dev<TYPE>(d.F);
    const uint32_t q8_row = d.F / 32 * Q8_0_BYTES;
    const uint32_t o0 = (blockIdx.x * 4 + wave) * RIF; // the grid covers every output once

    // round trip 1: everything that does not depend on the picks.  Every wave needs all of h (each
    // lane group one pick's row per round): fetched once per workgroup and shared through LDS --
    // a thousand waves each reading the same 18 KB made this round trip twice as long as the next.
    uint32_t eid[ROUNDS];
    float wt[ROUNDS];
#pragma unroll
    for (int q = 0; q < ROUNDS; q++) {
        const uint32_t s = q * GROUPS + grp;
        const uint32_t sc = s < d.k ? s : 0;
        eid[q] = sel->ids[sc];
        wt[q] = sel->w[sc];
    }
    float wsh = sel->w_shared;
    float res[RIF];
#pragma unroll
    for (int i = 0; i < RIF; i++) {
        if constexpr (RESID) res[i] = ra.p[min(o0 + i, d.H - 1)];
        else res[i] = 0.f;
    }
    const uint32_t h_quads = (d.k + 1) * d.F / 4;
    constexpr int HQ = 8; // quads per thread in flight: covers (16 + 1) * 1024 / 4 / 256 = 17 in three rounds
    const float4* hg = (const float4*)ws.h;
    float4 hq[HQ];
#pragma unroll
    for (int i = 0; i < HQ; i++) hq[i] = hg[min(threadIdx.x + 256u * i, h_quads - 1)];
    LaneW<QKK_Q8_0> wq[RIF];
#pragma unroll
    for (int i = 0; i < RIF; i++) wq[i].load(down_shexp + (size_t)min(o0 + i, d.H - 1) * q8_row, lir);
    fill_iq_tables(tab, g_iq3xxs_grid, threadIdx.x, 256);
#pragma unroll
    for (int i = 0; i < HQ; i++)
        if (threadIdx.x + 256u * i < h_quads) ((float4*)s_h)[threadIdx.x + 256u * i] = hq[i];
    for (uint32_t q4 = threadIdx.x + 256u * HQ; q4 < h_quads; q4 += 256u) ((float4*)s_h)[q4] = hg[q4]; // wide layers only

    // round trip 2
    LaneW<TYPE> w[RIF][ROUNDS];
#pragma unroll
    for (int q = 0; q < ROUNDS; q++) {
        const uint8_t* base = down_exps + (size_t)min(eid[q], d.E - 1) * d.H * row_bytes;
        if (q * GROUPS + grp >= (int)d.k) wt[q] = 0.f;
#pragma unroll
        for (int i = 0; i < RIF; i++) w[i][q].load(base + (size_t)min(o0 + i, d.H - 1) * row_bytes, lir);
    }
    if (grp != 0) wsh = 0.f;
    __syncthreads(); // h and the codebook in LDS
    XSlice hs[ROUNDS], hsh;
#pragma unroll
    for (int q = 0; q < ROUNDS; q++) {
        const uint32_t s = q * GROUPS + grp;
        load_xslice<TYPE>(hs[q], s_h + (size_t)(s < d.k ? s : 0) * d.F, lir);
    }
    load_xslice<QKK_Q8_0>(hsh, s_h + (size_t)d.k * d.F, lir);
    float hsum[ROUNDS][4];
#pragma unroll
    for (int q = 0; q < ROUNDS; q++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) a += hs[q].v[c * 8 + i];
            hsum[q][c] = a;
        }
#pragma unroll
    for (int i = 0; i < RIF; i++) {
        float acc = wsh * wq[i].dot(hsh, nullptr, nullptr, lir);
#pragma unroll
        for (int q = 0; q < ROUNDS; q++) acc += wt[q] * w[i][q].dot(hs[q], hsum[q], &tab, lir);
        acc = wave_sum(acc);
        if constexpr (RESID) acc += res[i];
        if (lane == 0 && o0 + i < d.H) y[o0 + i] = acc;
    }
}
template <int TYPE, int LPR, int ROUNDS, int RIF>
static void launch_down2(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y,
                         const MoeDims& d, const float* resid, uint32_t rows, hipStream_t st)
{
    const uint32_t waves = (d.H + RIF - 1) / RIF;
    const uint32_t lds = (d.k + 1) * d.F * 4; // h in LDS (at most 17 * 1024 floats = 68 KB)
    static bool raised = [] {
        for (const void* f : {(const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, false>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, false>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, false, true>,
                              (const void*)moe_down_kernel<TYPE, LPR, ROUNDS, RIF, true, true>})
            (void)hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 17 * 1024 * 4);
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
// Launches 1 and 2 for `rows` activation rows (grid.y); norm given (one row only): the variants with
// the RMS norm in front.
static void launch_route_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, qkk_sel* sel, const MoeDims& d,
                                uint32_t stages, const MoeNorm* norm, uint32_t rows, hipStream_t st)
{
    const uint8_t *gs = (const uint8_t*)L->gate_shexp, *us = (const uint8_t*)L->up_shexp;
    const uint8_t *ge = (const uint8_t*)L->gate_exps, *ue = (const uint8_t*)L->up_exps;
    const bool wide = d.H != 2048; // n_embd 4096
    const dim3 block(256);
    if (stages & QKK_STAGE_ROUTE) {
        const dim3 grid((d.E + 1 + d.F + 3) / 4, rows);
#define QK_ROUTE(K) hipLaunchKernelGGL(K, grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, ws, d)
#define QK_ROUTE_NORM(K) \
    hipLaunchKernelGGL(K, grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, ws, d, norm->w, norm->eps, \
                       AddArg<false>{})
#define QK_ROUTE_ADD(K) \
    hipLaunchKernelGGL(K, grid, block, 0, st, L->gate_inp, L->gate_inp_shexp, gs, us, X, ws, d, norm->w, norm->eps, \
                       AddArg<true>{norm->mix, norm->sum})
        if (norm && norm->mix) {
            if (!wide && rows > 1) QK_ROUTE_ADD((moe_route_norm_kernel<8, true, true>));
            else if (!wide) QK_ROUTE_ADD((moe_route_norm_kernel<8, false, true>));
            else if (rows > 1) QK_ROUTE_ADD((moe_route_norm_kernel<16, true, true>));
            else QK_ROUTE_ADD((moe_route_norm_kernel<16, false, true>));
        } else if (norm && rows > 1) {
            if (!wide) QK_ROUTE_NORM((moe_route_norm_kernel<8, true>));
            else QK_ROUTE_NORM((moe_route_norm_kernel<16, true>));
        } else if (norm) {
            if (!wide) QK_ROUTE_NORM((moe_route_norm_kernel<8, false>));
            else QK_ROUTE_NORM((moe_route_norm_kernel<16, false>));
        } else if (rows > 1) {
            if (!wide) QK_ROUTE((moe_route_kernel<8, true>));
            else QK_ROUTE((moe_route_kernel<16, true>));
        } else {
            if (!wide) QK_ROUTE((moe_route_kernel<8, false>));
            else QK_ROUTE((moe_route_kernel<16, false>));
        }
#undef QK_ROUTE
#undef QK_ROUTE_NORM
#undef QK_ROUTE_ADD
    }
    if (norm && norm->mix) X = norm->sum; // launch 2 reads the sum launch 1 stored
    if (stages & QKK_STAGE_GATEUP) {
        constexpr int GU_RIF = 4;
        const dim3 grid(wide ? (d.k * ((d.F + 1) / 2) + 3) / 4 : (d.k * ((d.F + GU_RIF - 1) / GU_RIF) + 3) / 4, rows);
#define QK_GATEUP(K) hipLaunchKernelGGL(K, grid, block, 0, st, ge, ue, X, ws, sel, d)
#define QK_GATEUP_NORM(K) hipLaunchKernelGGL(K, grid, block, 0, st, ge, ue, X, ws, sel, d, norm->w, norm->eps)
        if (norm && rows > 1) {
            if (!wide) QK_GATEUP_NORM((moe_gateup_norm_kernel<QKK_IQ3_XXS, 1, GU_RIF, true>));
            else QK_GATEUP_NORM((moe_gateup_norm_kernel<QKK_IQ3_XXS, 2, 2, true>));
        } else if (norm) {
            if (!wide) QK_GATEUP_NORM((moe_gateup_norm_kernel<QKK_IQ3_XXS, 1, GU_RIF, false>));
            else QK_GATEUP_NORM((moe_gateup_norm_kernel<QKK_IQ3_XXS, 2, 2, false>));
        } else if (rows > 1) {
            if (!wide) QK_GATEUP((moe_gateup_kernel<QKK_IQ3_XXS, 1, GU_RIF, true>));
            else QK_GATEUP((moe_gateup_kernel<QKK_IQ3_XXS, 2, 2, true>));
        } else {
            if (!wide) QK_GATEUP((moe_gateup_kernel<QKK_IQ3_XXS, 1, GU_RIF, false>));
            else QK_GATEUP((moe_gateup_kernel<QKK_IQ3_XXS, 2, 2, false>));
        }
#undef QK_GATEUP
#undef QK_GATEUP_NORM
    }
}

} // namespace lane

void lane_route_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, qkk_sel* sel, const MoeDims& d,
                       uint32_t stages, const MoeNorm* norm, uint32_t rows, hipStream_t st)
{
    lane::launch_route_gateup(L, X, ws, sel, d, stages, norm, rows, st);
}

void lane_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y, const MoeDims& d,
               const float* resid, uint32_t rows, hipStream_t st)
{
    if (L->down_type == QKK_IQ4_XS) lane::launch_down<QKK_IQ4_XS>(L, ws, sel, Y, d, resid, rows, st);
    else lane::launch_down<QKK_Q6_K>(L, ws, sel, Y, d, resid, rows, st);
}

} // namespace qk
