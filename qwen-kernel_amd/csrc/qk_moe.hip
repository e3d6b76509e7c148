// qk_moe.hip -- fused Qwen3-MoE decode step for gfx950.
//
// One activation row, three launches per step:
//   1. route:   router logits (F32 rows) + shared-expert gate dot + shared gate/up (Q8_0).
//   2. gate/up: every workgroup picks the top-n_used experts from the logits, then the routed
//               IQ3_XXS gate and up rows of the picks, SiLU gating -> h; writes the router record.
//   3. down:    routed down rows (IQ4_XS or Q6_K) weighted by the router, shared down row
//               (Q8_0) weighted by the sigmoid gate, summed into y.
// On this device a dependent memory access costs 2-3 us when the line is cold (each step
// touches a different layer's weights) while a kernel boundary costs well under 1 us, so each
// launch is arranged as two round trips at most and nothing synchronises inside a kernel.
// (A single-launch form with device-wide barriers was measured at ~5 us per barrier and
// dropped.)  Several rows go through the expert-major path in qk_moe_grouped.hip.
#include "qk_moe_common.h"

#include <mutex>

namespace qk {

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
                g += wg[i][p].dot_h(xs[p], &tab);
                u += wu[i][p].dot_h(xs[p], &tab);
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
                g += wg[i][p].dot_h(xs[p], &tab);
                u += wu[i][p].dot_h(xs[p], &tab);
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
    extern __shared__ __attribute__((aligned(16))) float s_h[]; // [(k+1)][F]: the gated activations of every pick
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

} // namespace qk

namespace qk {
int moe_grouped_launch(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                       uint32_t N, uint32_t stages, hipStream_t st, const MoeTail* tail);
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

constexpr uint32_t ROWWISE_MAX = QKK_ROWWISE_MAX; // rows up to which each row runs the one-row launches

// One row with the RMS norm in front (weights w) and the residual behind: see qkk_moe_layer_row.
struct MoeNorm {
    const float* w;
    float eps;
    const float* mix = nullptr; // the row is X + mix ...
    float* sum = nullptr;       // ... which launch 1 stores here for launches 2 and 3
};

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
    if (n_slots > ROWWISE_MAX) {
        if (norm) return fail(QKK_ESHAPE, "%s: %u rows exceed %u (use qkk_moe_decode_tail)", who, n_slots, ROWWISE_MAX);
        return moe_grouped_launch(L, X, Y, sel, workspace, n_slots, stages, st, tail);
    }
    const MoeWs ws = ws_carve(workspace, d, n_slots);

    launch_route_gateup(L, X, ws, sel, d, stages, norm, n_slots, st);
    if (stages & QKK_STAGE_DOWN) {
        // norm in front: the input row (with the mixer's output, if any) is the residual; Y may be X
        const float* resid = norm ? (norm->mix ? norm->sum : X) : nullptr;
        if (L->down_type == QKK_IQ4_XS) launch_down<QKK_IQ4_XS>(L, ws, sel, Y, d, resid, n_slots, st);
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
