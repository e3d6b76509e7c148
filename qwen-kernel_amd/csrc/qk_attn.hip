// qk_attn.hip -- the full-attention mixer's decode step: per-head q/k RMS norm, partial RoPE and
// KV-cache write (reference shaders/fa_prep_srv.comp:26-76), then attention of every slot's new
// token over its cached positions with the sigmoid output gate (reference
// shaders/fa_attn_srv.comp:27-95; split / grouped forms fa_attn_srv_split_gqa.comp,
// fa_attn_srv_reduce.comp; CPU mirror src/main.cpp:2138-2201).
//
// Shapes (the reference's: dh = 256, 16 query heads on 2 KV heads, 64 rotated dims):
//   qfull [slots][hQ][2*dh]   per head: dh query values, then dh output-gate pre-activations
//   kin, vin [slots][hKV][dh]
//   caches   [slots][hKV][tmax][dh] fp32, position-major per KV head
//   rope     [tmax][n_rot/2][2] (cos, sin), built by the caller (qkk_rope_table)
//   slot_pos [slots] device words: the position the new token is written at; n = pos + 1 keys
//
// Attention is bound by reading the cache: 2 * hKV * n * dh * 4 bytes per slot.  The G = hQ/hKV
// query heads that share a KV head are handled by ONE workgroup, so every K and V row is read once
// for all of them, and the positions are cut into ranges that run in parallel (two KV heads alone
// would leave 254 CUs idle; the host picks 8..64 ranges so that about two workgroups per CU
// result); a second launch folds the ranges' (max, sum, accumulator) triples in range order.  Which
// ranges hold keys is decided on the device from slot_pos, so the launch shape depends on the slot
// count and tmax only and a captured graph stays valid as the sequences grow.
#include "qk_device.h"
#include "qk_host.h"
#include "qk_mfma.h"

#include <math.h>
#include <stdlib.h>

#include <algorithm>

namespace qk {

constexpr uint32_t ATT_DH = 256;    // head size = workgroup size
constexpr uint32_t ATT_MAX_RANGES = 64; // position ranges per (slot, KV head), at most
constexpr uint32_t ATT_TILE = 64;   // positions scored per pass
constexpr uint32_t ATT_GMAX = 8;    // query heads per KV head
constexpr float ATT_FLOOR = -3.4e38f;

__device__ __forceinline__ uint32_t slot_position(const uint32_t* slot_pos, uint32_t rq, uint32_t tmax)
{
    return min(slot_pos[rq], tmax - 1u); // a position beyond the cache is clamped, never followed
}

// grid (hQ + 2*hKV, slots): workgroups [0,hQ) query heads, [hQ,hQ+hKV) key heads, then value heads.
__global__ __launch_bounds__(256) void attn_prep_kernel(const float* __restrict__ qfull, const float* __restrict__ kin,
                                                        const float* __restrict__ vin, const float* __restrict__ qn,
                                                        const float* __restrict__ kn, const float* __restrict__ rope,
                                                        const uint32_t* __restrict__ slot_pos, float* __restrict__ qhat,
                                                        float* __restrict__ kc, float* __restrict__ vc, uint32_t hQ,
                                                        uint32_t hKV, uint32_t n_rot, uint32_t tmax, float eps,
                                                        uint32_t own)
{
    __shared__ float s_v[ATT_DH];
    __shared__ float s_red[4];
    const uint32_t w = blockIdx.x, rq = blockIdx.y, t = threadIdx.x;
    const uint32_t pos = slot_position(slot_pos, rq, tmax);
    const size_t cq = (size_t)rq * own; // the cache row rq writes: its own, or the one all rows share
    if (w >= hQ + hKV) { // value head: copied into the cache
        const uint32_t h = w - hQ - hKV;
        vc[((cq * hKV + h) * tmax + pos) * ATT_DH + t] = vin[((size_t)rq * hKV + h) * ATT_DH + t];
        return;
    }
    const bool is_q = w < hQ;
    const uint32_t h = is_q ? w : w - hQ;
    const float v = is_q ? qfull[((size_t)rq * hQ + h) * 2 * ATT_DH + t] : kin[((size_t)rq * hKV + h) * ATT_DH + t];
    const float g = is_q ? qn[t] : kn[t];
    const float scale = 1.f / sqrtf(block_sum4(v * v, s_red) / (float)ATT_DH + eps);
    const float nv = v * scale * g;
    s_v[t] = nv;
    __syncthreads();
    float out = nv;
    const uint32_t half = n_rot / 2;
    if (t < n_rot) { // rotate the pair (j, j + half) by the position's angle for frequency j
        const uint32_t j = t < half ? t : t - half;
        const float c = rope[2 * ((size_t)pos * half + j)], s = rope[2 * ((size_t)pos * half + j) + 1];
        const float x0 = s_v[j], x1 = s_v[j + half];
        out = t < half ? x0 * c - x1 * s : x0 * s + x1 * c;
    }
    if (is_q) qhat[((size_t)rq * hQ + h) * ATT_DH + t] = out;
    else kc[((cq * hKV + h) * tmax + pos) * ATT_DH + t] = out;
}

// Partial results of one position range: per query head the running maximum, the sum of
// exp(score - maximum) and the exp-weighted sum of the value rows.
struct AttnWs {
    float* acc; // [slots][hQ][n_ranges][dh]
    float* ml;  // [slots][hQ][n_ranges][2]
};

// Eight floats as hi + lo halves (x = hi + lo to ~2^-22 of x): hi truncates x, lo rounds the exact rest.
struct HalfSplit {
    half8 hi, lo;
};
__device__ __forceinline__ HalfSplit split8(float4 a, float4 b)
{
    const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const auto hp = __builtin_amdgcn_cvt_pkrtz(x[2 * i], x[2 * i + 1]);
        const auto lp = __builtin_amdgcn_cvt_pkrtz(x[2 * i] - (float)hp[0], x[2 * i + 1] - (float)hp[1]);
        h[i] = __builtin_bit_cast(uint32_t, hp);
        l[i] = __builtin_bit_cast(uint32_t, lp);
    }
    HalfSplit r;
    r.hi = __builtin_bit_cast(half8, uint4{h[0], h[1], h[2], h[3]});
    r.lo = __builtin_bit_cast(half8, uint4{l[0], l[1], l[2], l[3]});
    return r;
}

// grid (n_ranges, hKV, slots), 256 threads.  The G query heads of one KV head over one position
// range, a tile of ATT_TILE positions at a time; wave w owns the tile's positions 16w .. 16w+15 and
// requests their K and V rows (32 pieces of 16 bytes per lane) before any arithmetic, so a tile
// costs one memory round trip.
//   scores  on the matrix cores: D[head][position] += Q[head][32 dims] . K[position][32 dims]
//           (v_mfma_f32_16x16x32_f16, heads padded to 16 with zeros), both operands split into
//           hi + lo halves and three products kept (hi.hi, hi.lo, lo.hi), so a score is exact to
//           ~2^-22 of its terms.  A K row's 256 dims are read by four lanes in pieces of 32 bytes,
//           full cache lines per wave instruction.  (Per-lane partial dot products folded across
//           the wave took ten times the vector instructions: one cross-lane sum per head and row.)
//   softmax running maximum and sum per head over the tile, in LDS.
//   values  a lane keeps 4 dims of every head's accumulator and adds its wave's 16 rows; the four
//           waves' accumulators are added through LDS at the end, in wave order.
__global__ __launch_bounds__(256) void attn_range_kernel(const float* __restrict__ qhat, const float* __restrict__ kc,
                                                         const float* __restrict__ vc,
                                                         const uint32_t* __restrict__ slot_pos, AttnWs ws, uint32_t hQ,
                                                         uint32_t hKV, uint32_t G, uint32_t tmax, uint32_t own)
{
    constexpr uint32_t RPW = ATT_TILE / 4; // rows per wave and tile (16: one MFMA column block)
    constexpr uint32_t KB = ATT_DH / 32;   // 32-dim blocks of a row
    __shared__ __attribute__((aligned(16))) half8 s_qh[KB][64], s_ql[KB][64]; // Q as the A operand, per lane
    __shared__ __attribute__((aligned(16))) float s_sc[ATT_GMAX][ATT_TILE];
    __shared__ float s_corr[ATT_GMAX], s_m[ATT_GMAX], s_l[ATT_GMAX];
    __shared__ __attribute__((aligned(16))) float s_acc[3][ATT_GMAX][ATT_DH]; // waves 1..3 hand theirs to wave 0
    const uint32_t n_ranges = gridDim.x, c = blockIdx.x, kv = blockIdx.y, rq = blockIdx.z, t = threadIdx.x;
    const uint32_t lane = t & 63u, wave = t >> 6, col = lane & 15u, quad = lane >> 4;
    const uint32_t n = slot_position(slot_pos, rq, tmax) + 1u;
    const uint32_t per = (tmax + n_ranges - 1) / n_ranges;
    const uint32_t p_begin = c * per, p_end = min(n, p_begin + per);
    if (p_begin >= n) return; // the whole workgroup: this range holds no key yet

    // Q operand: lane feeds A[head = col][dims 32*kb + 8*quad .. +7]; wave w prepares blocks 2w, 2w+1
#pragma unroll
    for (uint32_t i = 0; i < 2; i++) {
        const uint32_t kb = 2 * wave + i;
        float4 a = float4{0.f, 0.f, 0.f, 0.f}, b = a;
        if (col < G) {
            const float4* qrow = (const float4*)(qhat + ((size_t)rq * hQ + kv * G + col) * ATT_DH);
            a = qrow[kb * 8 + 2 * quad];
            b = qrow[kb * 8 + 2 * quad + 1];
        }
        const HalfSplit sp = split8(a, b);
        s_qh[kb][lane] = sp.hi;
        s_ql[kb][lane] = sp.lo;
    }
    if (t < ATT_GMAX) { s_m[t] = ATT_FLOOR; s_l[t] = 0.f; }
    const float qs = 1.f / sqrtf((float)ATT_DH);
    const float4* kbase = (const float4*)(kc + ((size_t)rq * own * hKV + kv) * tmax * ATT_DH);
    const float4* vbase = (const float4*)(vc + ((size_t)rq * own * hKV + kv) * tmax * ATT_DH);
    float4 acc[ATT_GMAX];
#pragma unroll
    for (uint32_t h = 0; h < ATT_GMAX; h++) acc[h] = float4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();

    for (uint32_t p0 = p_begin; p0 < p_end; p0 += ATT_TILE) {
        const uint32_t ts = min(ATT_TILE, p_end - p0);
        // rows beyond the tile repeat its last row (their scores are masked, their weights zero)
        const size_t krow = p0 + min(RPW * wave + col, ts - 1);
        float4 ka[KB], kb4[KB], v4[RPW];
#pragma unroll
        for (uint32_t kb = 0; kb < KB; kb++) {
            ka[kb] = kbase[krow * (ATT_DH / 4) + kb * 8 + 2 * quad];
            kb4[kb] = kbase[krow * (ATT_DH / 4) + kb * 8 + 2 * quad + 1];
        }
#pragma unroll
        for (uint32_t i = 0; i < RPW; i++)
            v4[i] = vbase[(size_t)(p0 + min(RPW * wave + i, ts - 1)) * (ATT_DH / 4) + lane];
        float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t kb = 0; kb < KB; kb++) {
            const HalfSplit k = split8(ka[kb], kb4[kb]);
            const half8 qh = s_qh[kb][lane], ql = s_ql[kb][lane];
            sc = mfma16x32(qh, k.hi, sc);
            sc = mfma16x32(qh, k.lo, sc);
            sc = mfma16x32(ql, k.hi, sc);
        }
        // D[4*quad + e][col]: head 4*quad + e, position 16*wave + col
#pragma unroll
        for (uint32_t e = 0; e < 4; e++)
            if (4 * quad + e < G) s_sc[4 * quad + e][RPW * wave + col] = sc[e] * qs;
        __syncthreads();
        // running maximum and sum per head: wave w folds heads w, w + 4 (lane = position of the tile)
        for (uint32_t h = wave; h < G; h += 4) {
            const float v = lane < ts ? s_sc[h][lane] : ATT_FLOOR;
            const float old_m = s_m[h];
            const float new_m = fmaxf(old_m, wave_max(v));
            const float e = lane < ts ? expf(v - new_m) : 0.f;
            const float tl = wave_sum(e);
            s_sc[h][lane] = e;
            if (lane == 0) {
                const float corr = expf(old_m - new_m);
                s_corr[h] = corr;
                s_m[h] = new_m;
                s_l[h] = s_l[h] * corr + tl;
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t h = 0; h < ATT_GMAX; h++) {
            if (h < G) { // uniform
                const float corr = s_corr[h];
                float4 a = float4{acc[h].x * corr, acc[h].y * corr, acc[h].z * corr, acc[h].w * corr};
#pragma unroll
                for (uint32_t i = 0; i < RPW; i += 4) { // the weights of positions beyond the tile are zero
                    const float4 w = *(const float4*)&s_sc[h][RPW * wave + i];
                    a.x += w.x * v4[i].x + w.y * v4[i + 1].x + w.z * v4[i + 2].x + w.w * v4[i + 3].x;
                    a.y += w.x * v4[i].y + w.y * v4[i + 1].y + w.z * v4[i + 2].y + w.w * v4[i + 3].y;
                    a.z += w.x * v4[i].z + w.y * v4[i + 1].z + w.z * v4[i + 2].z + w.w * v4[i + 3].z;
                    a.w += w.x * v4[i].w + w.y * v4[i + 1].w + w.z * v4[i + 2].w + w.w * v4[i + 3].w;
                }
                acc[h] = a;
            }
        }
        __syncthreads(); // the next tile overwrites the scores
    }
    // the four waves' accumulators, added in wave order
    if (wave > 0) {
#pragma unroll
        for (uint32_t h = 0; h < ATT_GMAX; h++)
            if (h < G) ((float4*)s_acc[wave - 1][h])[lane] = acc[h];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (uint32_t h = 0; h < ATT_GMAX; h++) {
            if (h < G) {
                float4 a = acc[h];
                for (uint32_t w = 0; w < 3; w++) {
                    const float4 b = ((const float4*)s_acc[w][h])[lane];
                    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
                }
                const size_t slot = ((size_t)rq * hQ + kv * G + h) * n_ranges + c;
                ((float4*)(ws.acc + slot * ATT_DH))[lane] = a;
                if (lane == 0) { ws.ml[2 * slot] = s_m[h]; ws.ml[2 * slot + 1] = s_l[h]; }
            }
        }
    }
}

// The same scan for TWO consecutive rows of a sequence (positions p, p + 1 of one slot) per
// workgroup: the second row's heads take the MFMA rows 8..15 that one row leaves empty, every cache
// row loaded serves both, and the later keys are masked per row.  grid (n_ranges, hKV, ceil(rows/2)).
__global__ __launch_bounds__(256) void attn_range_pair_kernel(const float* __restrict__ qhat, const float* __restrict__ kc,
                                                         const float* __restrict__ vc,
                                                         const uint32_t* __restrict__ slot_pos, AttnWs ws, uint32_t hQ,
                                                         uint32_t hKV, uint32_t G, uint32_t tmax, uint32_t rows)
{
    constexpr uint32_t RPW = ATT_TILE / 4; // rows per wave and tile (16: one MFMA column block)
    constexpr uint32_t KB = ATT_DH / 32;   // 32-dim blocks of a row
    constexpr uint32_t NH = 2 * ATT_GMAX;  // (row of the pair, head) = MFMA row 8 * row + head
    __shared__ __attribute__((aligned(16))) half8 s_qh[KB][64], s_ql[KB][64]; // Q as the A operand, per lane
    __shared__ __attribute__((aligned(16))) float s_sc[NH][ATT_TILE];
    __shared__ float s_corr[NH], s_m[NH], s_l[NH];
    __shared__ __attribute__((aligned(16))) float s_acc[3][ATT_GMAX][ATT_DH]; // waves 1..3 hand theirs to wave 0
    const uint32_t n_ranges = gridDim.x, c = blockIdx.x, kv = blockIdx.y, r0 = 2 * blockIdx.z, t = threadIdx.x;
    const bool two = r0 + 1 < rows; // the last pair of an odd row count has one row
    const uint32_t lane = t & 63u, wave = t >> 6, col = lane & 15u, quad = lane >> 4;
    const uint32_t n0 = slot_position(slot_pos, r0, tmax) + 1u;
    const uint32_t n1 = two ? slot_position(slot_pos, r0 + 1, tmax) + 1u : 0u;
    const uint32_t n = max(n0, n1);
    const uint32_t per = (tmax + n_ranges - 1) / n_ranges;
    const uint32_t p_begin = c * per, p_end = min(n, p_begin + per);
    if (p_begin >= n) return; // the whole workgroup: this range holds no key yet

    // Q operand: lane feeds A[head = col][dims 32*kb + 8*quad .. +7]; wave w prepares blocks 2w, 2w+1
#pragma unroll
    for (uint32_t i = 0; i < 2; i++) {
        const uint32_t kb = 2 * wave + i;
        float4 a = float4{0.f, 0.f, 0.f, 0.f}, b = a;
        const uint32_t qr = col >> 3, qhd = col & 7u;
        if (qhd < G && (qr == 0 || two)) {
            const float4* qrow = (const float4*)(qhat + ((size_t)(r0 + qr) * hQ + kv * G + qhd) * ATT_DH);
            a = qrow[kb * 8 + 2 * quad];
            b = qrow[kb * 8 + 2 * quad + 1];
        }
        const HalfSplit sp = split8(a, b);
        s_qh[kb][lane] = sp.hi;
        s_ql[kb][lane] = sp.lo;
    }
    if (t < NH) { s_m[t] = ATT_FLOOR; s_l[t] = 0.f; }
    const float qs = 1.f / sqrtf((float)ATT_DH);
    const float4* kbase = (const float4*)(kc + (size_t)kv * tmax * ATT_DH); // one slot's caches
    const float4* vbase = (const float4*)(vc + (size_t)kv * tmax * ATT_DH);
    float4 acc[NH];
#pragma unroll
    for (uint32_t h = 0; h < NH; h++) acc[h] = float4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();

    for (uint32_t p0 = p_begin; p0 < p_end; p0 += ATT_TILE) {
        const uint32_t ts = min(ATT_TILE, p_end - p0);
        // rows beyond the tile repeat its last row (their scores are masked, their weights zero)
        const size_t krow = p0 + min(RPW * wave + col, ts - 1);
        float4 ka[KB], kb4[KB], v4[RPW];
#pragma unroll
        for (uint32_t kb = 0; kb < KB; kb++) {
            ka[kb] = kbase[krow * (ATT_DH / 4) + kb * 8 + 2 * quad];
            kb4[kb] = kbase[krow * (ATT_DH / 4) + kb * 8 + 2 * quad + 1];
        }
#pragma unroll
        for (uint32_t i = 0; i < RPW; i++)
            v4[i] = vbase[(size_t)(p0 + min(RPW * wave + i, ts - 1)) * (ATT_DH / 4) + lane];
        float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t kb = 0; kb < KB; kb++) {
            const HalfSplit k = split8(ka[kb], kb4[kb]);
            const half8 qh = s_qh[kb][lane], ql = s_ql[kb][lane];
            sc = mfma16x32(qh, k.hi, sc);
            sc = mfma16x32(qh, k.lo, sc);
            sc = mfma16x32(ql, k.hi, sc);
        }
        // D[4*quad + e][col]: head 4*quad + e, position 16*wave + col
#pragma unroll
        for (uint32_t e = 0; e < 4; e++)
            if (((4 * quad + e) & 7u) < G) s_sc[4 * quad + e][RPW * wave + col] = sc[e] * qs;
        __syncthreads();
        // running maximum and sum per head: wave w folds heads w, w + 4 (lane = position of the tile)
        for (uint32_t h = wave; h < NH; h += 4) {
            if ((h & 7u) >= G || (h >= ATT_GMAX && !two)) continue; // the whole wave
            const bool live = lane < ts && p0 + lane < (h < ATT_GMAX ? n0 : n1); // a row sees the keys up to its own position
            const float v = live ? s_sc[h][lane] : ATT_FLOOR;
            const float old_m = s_m[h];
            const float new_m = fmaxf(old_m, wave_max(v));
            const float e = live ? expf(v - new_m) : 0.f;
            const float tl = wave_sum(e);
            s_sc[h][lane] = e;
            if (lane == 0) {
                const float corr = expf(old_m - new_m);
                s_corr[h] = corr;
                s_m[h] = new_m;
                s_l[h] = s_l[h] * corr + tl;
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t h = 0; h < NH; h++) {
            if ((h & 7u) < G && (h < ATT_GMAX || two)) { // uniform
                const float corr = s_corr[h];
                float4 a = float4{acc[h].x * corr, acc[h].y * corr, acc[h].z * corr, acc[h].w * corr};
#pragma unroll
                for (uint32_t i = 0; i < RPW; i += 4) { // the weights of positions beyond the tile are zero
                    const float4 w = *(const float4*)&s_sc[h][RPW * wave + i];
                    a.x += w.x * v4[i].x + w.y * v4[i + 1].x + w.z * v4[i + 2].x + w.w * v4[i + 3].x;
                    a.y += w.x * v4[i].y + w.y * v4[i + 1].y + w.z * v4[i + 2].y + w.w * v4[i + 3].y;
                    a.z += w.x * v4[i].z + w.y * v4[i + 1].z + w.z * v4[i + 2].z + w.w * v4[i + 3].z;
                    a.w += w.x * v4[i].w + w.y * v4[i + 1].w + w.z * v4[i + 2].w + w.w * v4[i + 3].w;
                }
                acc[h] = a;
            }
        }
        __syncthreads(); // the next tile overwrites the scores
    }
    // the four waves' accumulators, added in wave order; one row of the pair at a time through s_acc
#pragma unroll
    for (uint32_t half = 0; half < 2; half++) {
        if (half == 1 && !two) break; // the whole workgroup
        if (wave > 0) {
#pragma unroll
            for (uint32_t h = 0; h < ATT_GMAX; h++)
                if (h < G) ((float4*)s_acc[wave - 1][h])[lane] = acc[half * ATT_GMAX + h];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (uint32_t h = 0; h < ATT_GMAX; h++) {
                if (h < G) {
                    float4 a = acc[half * ATT_GMAX + h];
                    for (uint32_t w = 0; w < 3; w++) {
                        const float4 b = ((const float4*)s_acc[w][h])[lane];
                        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
                    }
                    const size_t slot = ((size_t)(r0 + half) * hQ + kv * G + h) * n_ranges + c;
                    ((float4*)(ws.acc + slot * ATT_DH))[lane] = a;
                    if (lane == 0) { ws.ml[2 * slot] = s_m[half * ATT_GMAX + h]; ws.ml[2 * slot + 1] = s_l[half * ATT_GMAX + h]; }
                }
            }
        }
        __syncthreads(); // s_acc is reused by the second row
    }
}

// ---- sixteen consecutive rows of a sequence per workgroup (prompt prefill) ----------------------
// Stands for the reference's blocked prefill attention (shaders/fa_attn_batch_coopmat.comp:58-183: 16
// queries x 64 keys per iteration, both products on cooperative matrices).  grid (n_ranges, hKV *
// ceil(G / 4), ceil(rows / 16)), 256 threads.  One workgroup takes SIXTEEN rows and FOUR of the G query
// heads of one KV head over one position range, so every cached K and V row is fetched once for 64
// query rows (the pair kernel above fetches it once per two rows of all G heads).  Wave w owns one
// head from end to end -- scores, softmax, values -- so the running maximum, the sum and the
// rescaling of the accumulators stay inside the wave (a query row's 16 scores of a key block lie in
// the 16 lanes of one DPP row):
//   K tile   64 keys as halves hi + lo in LDS, row-major (the B operand of Q.K^T reads 8 dims = 16 bytes);
//   scores   S[query][key]: 4 key blocks x 8 steps of 32 dims x 3 products (hi.hi, hi.lo, lo.hi);
//            Q (pre-scaled by 1/sqrt(dh), a power of two) stays in registers as hi + lo;
//   softmax  in the MFMA output layout: lane (quad, col) holds rows 4*quad + e, key 16*kb + col;
//   P        hi + lo halves through a wave-private LDS area into the A operand layout;
//   V tile   in the K tile's place, TRANSPOSED ([dim][key]): the B operand of P.V reads 8 keys = 16 bytes;
//   values   O[query][dim] += P.V: 16 dim blocks x 2 steps of 32 keys x 3 products, accumulators in
//            registers (64), rescaled in place by exp(old max - new max).
// Later keys are masked per row (a key is visible to row i iff it lies below pos[i] + 1), so any
// positions work.  The (max, sum, accumulator) triples go to the same workspace as the other range
// kernels' and attn_fold_kernel finishes the rows.
constexpr uint32_t BLK_Q = 16;                    // rows per workgroup
constexpr uint32_t BLK_KP = ATT_DH * 2 + 16;      // K tile row pitch in bytes (halves): 528
constexpr uint32_t BLK_VP = ATT_TILE * 2 + 16;    // V^T tile row pitch in bytes: 144
constexpr uint32_t BLK_PP = ATT_TILE * 2 + 16;    // P row pitch in bytes: 144
constexpr uint32_t BLK_KV_BYTES = 2 * ATT_DH * BLK_VP;       // hi + lo of the larger tile (V^T): 73,728
constexpr uint32_t BLK_P_BYTES = 2 * BLK_Q * BLK_PP;         // per wave: (hi, lo) x 16 rows: 4,608
constexpr uint32_t BLK_LDS = BLK_KV_BYTES + 4 * BLK_P_BYTES; // 92,160
static_assert(2 * ATT_TILE * BLK_KP <= BLK_KV_BYTES, "the K tile fits the V tile's area");

typedef uint16_t __attribute__((may_alias)) lds_u16;
typedef uint4 __attribute__((may_alias)) lds_u128;
typedef uint2 __attribute__((may_alias)) lds_u64;

__device__ __forceinline__ float dpp_row_max(float v) // maximum over the 16 lanes of a DPP row, in every lane
{
    v = fmaxf(v, dpp_f<DPP_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
    return fmaxf(v, dpp_f<DPP_MIRROR>(v));
}

__global__ __launch_bounds__(256) void attn_block_kernel(const float* __restrict__ qhat, const float* __restrict__ kc,
                                                         const float* __restrict__ vc,
                                                         const uint32_t* __restrict__ slot_pos, AttnWs ws, uint32_t hQ,
                                                         uint32_t hKV, uint32_t G, uint32_t tmax, uint32_t rows)
{
    QK_DYN_LDS(uint8_t, s_blk);
    constexpr uint32_t KS = ATT_DH / 32; // 32-dim steps of a row
    const uint32_t n_ranges = gridDim.x, c = blockIdx.x, r0 = BLK_Q * blockIdx.z, t = threadIdx.x;
    const uint32_t hgroups = (G + 3) / 4, kv = blockIdx.y / hgroups, hg = blockIdx.y % hgroups;
    const uint32_t lane = t & 63u, wave = t >> 6, col = lane & 15u, quad = lane >> 4;
    const uint32_t nq = min(BLK_Q, rows - r0);
    // keys visible to the rows this lane holds in the output layout (rows 4 * quad + e), and to any row
    uint32_t n_row[4], n_max = 0;
#pragma unroll
    for (uint32_t e = 0; e < 4; e++) n_row[e] = 4 * quad + e < nq ? slot_position(slot_pos, r0 + 4 * quad + e, tmax) + 1u : 0u;
    for (uint32_t i = 0; i < nq; i++) n_max = max(n_max, slot_position(slot_pos, r0 + i, tmax) + 1u);
    const uint32_t per = (tmax + n_ranges - 1) / n_ranges;
    const uint32_t p_begin = c * per, p_end = min(n_max, p_begin + per);
    if (p_begin >= n_max) return; // the whole workgroup: this range holds no key of any row

    uint8_t* s_kv = s_blk;                                    // K tile (hi, lo), then the V^T tile (hi, lo)
    uint8_t* s_p = s_blk + BLK_KV_BYTES + wave * BLK_P_BYTES; // this wave's P: [hi, lo][row][key]
    const uint32_t hq_in = 4 * hg + wave;                     // this wave's head among the G of the KV head
    const bool has = hq_in < G;                               // uniform per wave; a wave without a head still stages tiles
    const uint32_t head = kv * G + min(hq_in, G - 1);

    // Q operand: lane feeds A[row = col][dims 32 * ks + 8 * quad .. + 7], scaled by 1/sqrt(dh)
    half8 qh[KS], ql[KS];
    const float qs = 1.f / sqrtf((float)ATT_DH);
#pragma unroll
    for (uint32_t ks = 0; ks < KS; ks++) {
        float4 a = float4{0.f, 0.f, 0.f, 0.f}, b = a;
        if (col < nq) {
            const float4* qrow = (const float4*)(qhat + ((size_t)(r0 + col) * hQ + head) * ATT_DH);
            a = qrow[ks * 8 + 2 * quad];
            b = qrow[ks * 8 + 2 * quad + 1];
        }
        const HalfSplit sp = split8(float4{a.x * qs, a.y * qs, a.z * qs, a.w * qs},
                                    float4{b.x * qs, b.y * qs, b.z * qs, b.w * qs});
        qh[ks] = sp.hi;
        ql[ks] = sp.lo;
    }
    float4v o[ATT_DH / 16];
    float m_run[4], l_run[4];
#pragma unroll
    for (uint32_t db = 0; db < ATT_DH / 16; db++) o[db] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (uint32_t e = 0; e < 4; e++) { m_run[e] = ATT_FLOOR; l_run[e] = 0.f; }
    const float4* kbase = (const float4*)(kc + (size_t)kv * tmax * ATT_DH); // one slot's caches
    const float4* vbase = (const float4*)(vc + (size_t)kv * tmax * ATT_DH);

    // staging of a tile: wave w fetches the rows 16 w .. 16 w + 15
    //   K: one row per instruction, lane = 4 dims (a row is 64 consecutive float4)
    //   V: lane = (key 16 w + lane % 16, dims 4 * (lane / 16 + 4 * i)), so that the transposed 2-byte stores of
    //      16 lanes fall on consecutive keys
    float4 stage[16];
    auto fetch_k = [&](uint32_t p0, uint32_t ts) {
#pragma unroll
        for (uint32_t i = 0; i < 16; i++)
            stage[i] = kbase[(size_t)(p0 + min(16 * wave + i, ts - 1)) * (ATT_DH / 4) + lane];
    };
    auto fetch_v = [&](uint32_t p0, uint32_t ts) {
        const size_t row = p0 + min(16 * wave + col, ts - 1);
#pragma unroll
        for (uint32_t i = 0; i < 16; i++) stage[i] = vbase[row * (ATT_DH / 4) + quad + 4 * i];
    };
    auto split4 = [](float4 v, uint2& hi, uint2& lo) {
        const auto h0 = __builtin_amdgcn_cvt_pkrtz(v.x, v.y), h1 = __builtin_amdgcn_cvt_pkrtz(v.z, v.w);
        const auto l0 = __builtin_amdgcn_cvt_pkrtz(v.x - (float)h0[0], v.y - (float)h0[1]);
        const auto l1 = __builtin_amdgcn_cvt_pkrtz(v.z - (float)h1[0], v.w - (float)h1[1]);
        hi = uint2{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1)};
        lo = uint2{__builtin_bit_cast(uint32_t, l0), __builtin_bit_cast(uint32_t, l1)};
    };

    fetch_k(p_begin, min(ATT_TILE, p_end - p_begin));
    for (uint32_t p0 = p_begin; p0 < p_end; p0 += ATT_TILE) {
        const uint32_t ts = min(ATT_TILE, p_end - p0);
        __syncthreads(); // the previous tile's V has been consumed
        // K tile: [key][dim] halves, hi at 0, lo behind it
#pragma unroll
        for (uint32_t i = 0; i < 16; i++) {
            uint2 hi, lo;
            split4(stage[i], hi, lo);
            const uint32_t at = (16 * wave + i) * BLK_KP + lane * 8;
            *(lds_u64*)(s_kv + at) = hi;
            *(lds_u64*)(s_kv + ATT_TILE * BLK_KP + at) = lo;
        }
        fetch_v(p0, ts); // in flight during the scores
        __syncthreads();

        if (has) {
            float4v sc[4];
#pragma unroll
            for (uint32_t kb = 0; kb < 4; kb++) {
                sc[kb] = float4v{0.f, 0.f, 0.f, 0.f};
                const uint32_t at = (16 * kb + col) * BLK_KP + quad * 16;
#pragma unroll
                for (uint32_t ks = 0; ks < KS; ks++) {
                    const half8 kh = __builtin_bit_cast(half8, *(const lds_u128*)(s_kv + at + ks * 64));
                    const half8 kl = __builtin_bit_cast(half8, *(const lds_u128*)(s_kv + ATT_TILE * BLK_KP + at + ks * 64));
                    sc[kb] = mfma16x32(qh[ks], kh, sc[kb]);
                    sc[kb] = mfma16x32(qh[ks], kl, sc[kb]);
                    sc[kb] = mfma16x32(ql[ks], kh, sc[kb]);
                }
            }
            // sc[kb][e]: row 4 * quad + e, key p0 + 16 * kb + col
#pragma unroll
            for (uint32_t e = 0; e < 4; e++) {
                float mx = ATT_FLOOR;
                bool vis[4];
#pragma unroll
                for (uint32_t kb = 0; kb < 4; kb++) {
                    const uint32_t key = p0 + 16 * kb + col;
                    vis[kb] = key < p_end && key < n_row[e];
                    if (vis[kb]) mx = fmaxf(mx, sc[kb][e]);
                }
                const float new_m = fmaxf(m_run[e], dpp_row_max(mx));
                const float corr = expf(m_run[e] - new_m);
                float sum = 0.f;
#pragma unroll
                for (uint32_t kb = 0; kb < 4; kb++) {
                    const float pv = vis[kb] ? expf(sc[kb][e] - new_m) : 0.f;
                    sum += pv;
                    const _Float16 hi = (_Float16)pv;   // round to nearest; the rest is exact in fp32
                    const _Float16 lo = (_Float16)(pv - (float)hi);
                    const uint32_t at = (4 * quad + e) * BLK_PP + (16 * kb + col) * 2;
                    *(lds_u16*)(s_p + at) = __builtin_bit_cast(uint16_t, hi);
                    *(lds_u16*)(s_p + BLK_Q * BLK_PP + at) = __builtin_bit_cast(uint16_t, lo);
                }
                l_run[e] = l_run[e] * corr + group_sum<16>(sum);
                m_run[e] = new_m;
#pragma unroll
                for (uint32_t db = 0; db < ATT_DH / 16; db++) o[db][e] *= corr;
            }
        }
        __syncthreads(); // every wave has read the K tile
        // V^T tile: [dim][key] halves, hi at 0, lo behind it
#pragma unroll
        for (uint32_t i = 0; i < 16; i++) {
            uint2 hi, lo;
            split4(stage[i], hi, lo);
            const uint32_t d0 = 4 * (quad + 4 * i), at = d0 * BLK_VP + (16 * wave + col) * 2;
            *(lds_u16*)(s_kv + at) = (uint16_t)(hi.x & 0xFFFFu);
            *(lds_u16*)(s_kv + at + BLK_VP) = (uint16_t)(hi.x >> 16);
            *(lds_u16*)(s_kv + at + 2 * BLK_VP) = (uint16_t)(hi.y & 0xFFFFu);
            *(lds_u16*)(s_kv + at + 3 * BLK_VP) = (uint16_t)(hi.y >> 16);
            *(lds_u16*)(s_kv + ATT_DH * BLK_VP + at) = (uint16_t)(lo.x & 0xFFFFu);
            *(lds_u16*)(s_kv + ATT_DH * BLK_VP + at + BLK_VP) = (uint16_t)(lo.x >> 16);
            *(lds_u16*)(s_kv + ATT_DH * BLK_VP + at + 2 * BLK_VP) = (uint16_t)(lo.y & 0xFFFFu);
            *(lds_u16*)(s_kv + ATT_DH * BLK_VP + at + 3 * BLK_VP) = (uint16_t)(lo.y >> 16);
        }
        if (p0 + ATT_TILE < p_end) fetch_k(p0 + ATT_TILE, min(ATT_TILE, p_end - p0 - ATT_TILE)); // in flight during the values
        __syncthreads();

        // values: O[row][dim] += P[row][key] . V[key][dim]; the weights of masked keys are zero
        if (has) {
            half8 pa_h[2], pa_l[2];
#pragma unroll
            for (uint32_t ks = 0; ks < 2; ks++) { // A[row = col][keys 32 * ks + 8 * quad .. + 7]
                const uint32_t at = col * BLK_PP + (32 * ks + 8 * quad) * 2;
                pa_h[ks] = __builtin_bit_cast(half8, *(const lds_u128*)(s_p + at));
                pa_l[ks] = __builtin_bit_cast(half8, *(const lds_u128*)(s_p + BLK_Q * BLK_PP + at));
            }
#pragma unroll
            for (uint32_t db = 0; db < ATT_DH / 16; db++) {
#pragma unroll
                for (uint32_t ks = 0; ks < 2; ks++) { // B[keys 32 * ks + 8 * quad .. + 7][dim = 16 * db + col]
                    const uint32_t at = (16 * db + col) * BLK_VP + (32 * ks + 8 * quad) * 2;
                    const half8 vh = __builtin_bit_cast(half8, *(const lds_u128*)(s_kv + at));
                    const half8 vl = __builtin_bit_cast(half8, *(const lds_u128*)(s_kv + ATT_DH * BLK_VP + at));
                    o[db] = mfma16x32(pa_h[ks], vh, o[db]);
                    o[db] = mfma16x32(pa_h[ks], vl, o[db]);
                    o[db] = mfma16x32(pa_l[ks], vh, o[db]);
                }
            }
        }
    }
    // the range's triples: o[db][e] is row 4 * quad + e, dim 16 * db + col
    if (!has) return;
#pragma unroll
    for (uint32_t e = 0; e < 4; e++) {
        const uint32_t i = 4 * quad + e;
        if (i >= nq) continue;
        const size_t slot = ((size_t)(r0 + i) * hQ + head) * n_ranges + c;
#pragma unroll
        for (uint32_t db = 0; db < ATT_DH / 16; db++) ws.acc[slot * ATT_DH + 16 * db + col] = o[db][e];
        if (col == 0) { ws.ml[2 * slot] = m_run[e]; ws.ml[2 * slot + 1] = l_run[e]; }
    }
}

// grid (hQ, slots), 256 threads: folds the ranges of one query head in range order, divides by the
// sum and applies the output gate sigmoid(qfull[head][dh + t]).  Wave w adds the ranges w, w+4, ...
// (a lane 4 dims, eight ranges requested at a time); the waves' sums are added in wave order.
__global__ __launch_bounds__(256) void attn_fold_kernel(AttnWs ws, const float* __restrict__ qfull,
                                                        const uint32_t* __restrict__ slot_pos, float* __restrict__ att,
                                                        uint32_t hQ, uint32_t tmax, uint32_t n_ranges_all)
{
    __shared__ float s_f[ATT_MAX_RANGES], s_lf[ATT_MAX_RANGES];
    __shared__ __attribute__((aligned(16))) float s_o[4][ATT_DH];
    const uint32_t h = blockIdx.x, rq = blockIdx.y, t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const uint32_t n = slot_position(slot_pos, rq, tmax) + 1u;
    const uint32_t per = (tmax + n_ranges_all - 1) / n_ranges_all;
    const uint32_t n_ranges = min(n_ranges_all, (n + per - 1) / per); // the ranges that hold keys
    const size_t base = ((size_t)rq * hQ + h) * n_ranges_all;
    const float g = qfull[((size_t)rq * hQ + h) * 2 * ATT_DH + ATT_DH + t];
    float my_m = ATT_FLOOR, my_l = 0.f;
    if (t < n_ranges) { my_m = ws.ml[2 * (base + t)]; my_l = ws.ml[2 * (base + t) + 1]; }
    if (t < ATT_MAX_RANGES) s_f[t] = my_m;
    __syncthreads();
    float m = ATT_FLOOR;
    for (uint32_t c = 0; c < n_ranges; c++) m = fmaxf(m, s_f[c]);
    __syncthreads();
    if (t < n_ranges) {
        const float f = expf(my_m - m);
        s_f[t] = f;
        s_lf[t] = my_l * f;
    }
    __syncthreads();
    float l = 0.f;
    for (uint32_t c = 0; c < n_ranges; c++) l += s_lf[c];
    float4 o = float4{0.f, 0.f, 0.f, 0.f};
    for (uint32_t c0 = wave; c0 < n_ranges; c0 += 32) {
        float4 a[8];
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) {
            const uint32_t c = min(c0 + 4 * i, n_ranges - 1);
            a[i] = ((const float4*)(ws.acc + (base + c) * ATT_DH))[lane];
        }
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) {
            const float f = c0 + 4 * i < n_ranges ? s_f[c0 + 4 * i] : 0.f;
            o.x += a[i].x * f; o.y += a[i].y * f; o.z += a[i].z * f; o.w += a[i].w * f;
        }
    }
    ((float4*)s_o[wave])[lane] = o;
    __syncthreads();
    const float tot = ((s_o[0][t] + s_o[1][t]) + s_o[2][t]) + s_o[3][t];
    att[((size_t)rq * hQ + h) * ATT_DH + t] = (tot / l) * (1.f / (1.f + expf(-g)));
}

static int check_shape(const char* who, uint32_t n_slots, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax)
{
    if (n_slots < 1 || n_slots > 65535) return fail(QKK_ESHAPE, "%s: %u slots outside 1..65535", who, n_slots);
    if (dh != ATT_DH) return fail(QKK_ESHAPE, "%s: head size %u not supported (256)", who, dh);
    if (hKV < 1 || hQ < hKV || hQ % hKV || hQ / hKV > ATT_GMAX || hQ > 4096)
        return fail(QKK_ESHAPE, "%s: %u query heads on %u KV heads not supported (a multiple, at most %u per KV head)", who,
                    hQ, hKV, ATT_GMAX);
    if (tmax < 1 || tmax > (1u << 24)) return fail(QKK_ESHAPE, "%s: tmax %u outside 1..2^24", who, tmax);
    return QKK_OK;
}

} // namespace qk

using namespace qk;

extern "C" {

int qkk_rope_table(float* rope_host, uint32_t tmax, uint32_t n_rot, float freq_base)
{
    if (!rope_host) return fail(QKK_EINVAL, "qkk_rope_table: null pointer");
    if (n_rot < 2 || n_rot % 2 || tmax < 1) return fail(QKK_ESHAPE, "qkk_rope_table: n_rot must be even and tmax positive");
    const uint32_t half = n_rot / 2;
    for (uint32_t p = 0; p < tmax; p++)
        for (uint32_t j = 0; j < half; j++) { // reference src/main.cpp:2011-2020, all in float
            const float th = (float)p * powf(freq_base, -2.f * (float)j / (float)n_rot);
            rope_host[2 * ((size_t)p * half + j)] = cosf(th);
            rope_host[2 * ((size_t)p * half + j) + 1] = sinf(th);
        }
    return QKK_OK;
}

// rows of their own caches (own = 1: decode, one row per slot) or of one cache (own = 0: consecutive
// positions of one slot)
static int attn_prep_impl(const char* who, const float* qfull, const float* kin, const float* vin, const float* q_norm_w,
                          const float* k_norm_w, const float* rope, const uint32_t* slot_pos, float* qhat, float* k_cache,
                          float* v_cache, uint32_t rows, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t n_rot,
                          uint32_t tmax, float eps, uint32_t own, void* stream)
{
    if (!qfull || !kin || !vin || !q_norm_w || !k_norm_w || !rope || !slot_pos || !qhat || !k_cache || !v_cache)
        return fail(QKK_EINVAL, "%s: null pointer", who);
    if (int rc = check_shape(who, rows, hQ, hKV, dh, tmax)) return rc;
    if (n_rot < 2 || n_rot % 2 || n_rot > dh) return fail(QKK_ESHAPE, "%s: n_rot %u must be even, 2..%u", who, n_rot, dh);
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "%s: eps must be non-negative", who);
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(attn_prep_kernel, dim3(hQ + 2 * hKV, rows), dim3(256), 0, as_stream(stream), qfull, kin, vin,
                       q_norm_w, k_norm_w, rope, slot_pos, qhat, k_cache, v_cache, hQ, hKV, n_rot, tmax, eps, own);
    return check_launch(who);
}

int qkk_attn_prep(const float* qfull, const float* kin, const float* vin, const float* q_norm_w, const float* k_norm_w,
                  const float* rope, const uint32_t* slot_pos, float* qhat, float* k_cache, float* v_cache,
                  uint32_t n_slots, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t n_rot, uint32_t tmax, float eps,
                  void* stream)
{
    return attn_prep_impl("qkk_attn_prep", qfull, kin, vin, q_norm_w, k_norm_w, rope, slot_pos, qhat, k_cache, v_cache,
                          n_slots, hQ, hKV, dh, n_rot, tmax, eps, 1, stream);
}

int qkk_attn_prep_seq(const float* qfull, const float* kin, const float* vin, const float* q_norm_w, const float* k_norm_w,
                      const float* rope, const uint32_t* positions, float* qhat, float* k_cache, float* v_cache,
                      uint32_t n_pos, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t n_rot, uint32_t tmax, float eps,
                      void* stream)
{
    return attn_prep_impl("qkk_attn_prep_seq", qfull, kin, vin, q_norm_w, k_norm_w, rope, positions, qhat, k_cache, v_cache,
                          n_pos, hQ, hKV, dh, n_rot, tmax, eps, 0, stream);
}

// Position ranges a launch over `rows` rows uses at most: the more rows, the fewer ranges are needed
// to fill the chip (two workgroups per CU over rows x KV heads; 512 CUs assumed for the bound).
static uint32_t max_ranges(uint32_t rows) { return std::min(ATT_MAX_RANGES, std::max(8u, 512u / rows)); }

size_t qkk_attn_workspace_bytes(uint32_t n_slots, uint32_t hQ, uint32_t dh)
{
    if (!n_slots || !hQ || !dh) return 0;
    return (size_t)n_slots * hQ * max_ranges(n_slots) * ((size_t)dh + 2) * sizeof(float) + 256;
}

static int attn_decode_impl(const char* who, const float* qhat, const float* k_cache, const float* v_cache,
                            const float* qfull, const uint32_t* slot_pos, float* att, void* workspace,
                            size_t workspace_bytes, uint32_t rows, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax,
                            uint32_t own, void* stream)
{
    if (!qhat || !k_cache || !v_cache || !qfull || !slot_pos || !att || !workspace) return fail(QKK_EINVAL, "%s: null pointer", who);
    if (int rc = check_shape(who, rows, hQ, hKV, dh, tmax)) return rc;
    if (!aligned16(qhat) || !aligned16(k_cache) || !aligned16(v_cache) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return fail(QKK_EINVAL, "%s: qhat and the caches must be 16-byte, workspace 256-byte aligned", who);
    if (workspace_bytes < qkk_attn_workspace_bytes(rows, hQ, dh))
        return fail(QKK_EWORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
                    qkk_attn_workspace_bytes(rows, hQ, dh));
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    // two workgroups per CU over the (row, KV head) pairs, 8..64 ranges each: 16 slots x 4096 positions
    // measured 4.5 TB/s with 16 ranges, 4.2 with 32, 3.1 with 128 (the partial results are traffic too);
    // one slot 0.98 TB/s with 64 ranges, 0.80 with 32
    uint32_t n_ranges = std::min(max_ranges(rows), std::max(8u, persistent_blocks() / 2 / (rows * hKV)));
    // the "attn_block" switch: three or more consecutive rows of one slot go in blocks of sixteen rows instead of
    // pairs; one workgroup per CU (LDS), so about as many (block, KV head, range) triples as there are CUs
    const bool blocked = own == 0 && rows >= 3 && options().attn_block;
    const uint32_t blocks = (rows + BLK_Q - 1) / BLK_Q;
    const uint32_t hgroups = (hQ / hKV + 3) / 4; // four query heads of a KV head per workgroup
    if (blocked) n_ranges = std::min(max_ranges(rows), std::max(1u, persistent_blocks() / 4 / (blocks * hKV * hgroups)));
    AttnWs ws;
    ws.acc = (float*)workspace;
    ws.ml = ws.acc + (size_t)rows * hQ * n_ranges * ATT_DH;
    if (blocked) {
        static bool once = ((void)hipFuncSetAttribute((const void*)attn_block_kernel,
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)BLK_LDS), true);
        (void)once;
        hipLaunchKernelGGL(attn_block_kernel, dim3(n_ranges, hKV * hgroups, blocks), dim3(256), BLK_LDS, st, qhat, k_cache, v_cache,
                           slot_pos, ws, hQ, hKV, hQ / hKV, tmax, rows);
    } else if (own == 0 && rows >= 2)
        hipLaunchKernelGGL(attn_range_pair_kernel, dim3(n_ranges, hKV, (rows + 1) / 2), dim3(256), 0, st, qhat, k_cache,
                           v_cache, slot_pos, ws, hQ, hKV, hQ / hKV, tmax, rows);
    else
        hipLaunchKernelGGL(attn_range_kernel, dim3(n_ranges, hKV, rows), dim3(256), 0, st, qhat, k_cache, v_cache, slot_pos,
                           ws, hQ, hKV, hQ / hKV, tmax, own);
    hipLaunchKernelGGL(attn_fold_kernel, dim3(hQ, rows), dim3(256), 0, st, ws, qfull, slot_pos, att, hQ, tmax, n_ranges);
    return check_launch(who);
}

int qkk_attn_decode(const float* qhat, const float* k_cache, const float* v_cache, const float* qfull,
                    const uint32_t* slot_pos, float* att, void* workspace, size_t workspace_bytes, uint32_t n_slots,
                    uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax, void* stream)
{
    return attn_decode_impl("qkk_attn_decode", qhat, k_cache, v_cache, qfull, slot_pos, att, workspace, workspace_bytes,
                            n_slots, hQ, hKV, dh, tmax, 1, stream);
}

int qkk_attn_seq(const float* qhat, const float* k_cache, const float* v_cache, const float* qfull,
                 const uint32_t* positions, float* att, void* workspace, size_t workspace_bytes, uint32_t n_pos, uint32_t hQ,
                 uint32_t hKV, uint32_t dh, uint32_t tmax, void* stream)
{
    return attn_decode_impl("qkk_attn_seq", qhat, k_cache, v_cache, qfull, positions, att, workspace, workspace_bytes, n_pos,
                            hQ, hKV, dh, tmax, 0, stream);
}

} // extern "C"
