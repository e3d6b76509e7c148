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
// for all of them, and the positions are cut into ATT_CHUNKS ranges that run in parallel (two KV
// heads alone would leave 254 CUs idle); a second launch folds the ranges' (max, sum, accumulator)
// triples in range order.  Which ranges hold keys is decided on the device from slot_pos, so the
// launch shape depends on tmax only and a captured graph stays valid as the sequences grow.
#include "qk_device.h"
#include "qk_host.h"

#include <math.h>

namespace qk {

constexpr uint32_t ATT_DH = 256;    // head size = workgroup size
constexpr uint32_t ATT_CHUNKS = 64; // position ranges per (slot, KV head)
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
                                                        uint32_t hKV, uint32_t n_rot, uint32_t tmax, float eps)
{
    __shared__ float s_v[ATT_DH];
    __shared__ float s_red[4];
    const uint32_t w = blockIdx.x, rq = blockIdx.y, t = threadIdx.x;
    const uint32_t pos = slot_position(slot_pos, rq, tmax);
    if (w >= hQ + hKV) { // value head: copied into the cache
        const uint32_t h = w - hQ - hKV;
        vc[(((size_t)rq * hKV + h) * tmax + pos) * ATT_DH + t] = vin[((size_t)rq * hKV + h) * ATT_DH + t];
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
    else kc[(((size_t)rq * hKV + h) * tmax + pos) * ATT_DH + t] = out;
}

// Partial results of one position range: per query head the running maximum, the sum of
// exp(score - maximum) and the exp-weighted sum of the value rows.
struct AttnWs {
    float* acc; // [slots][hQ][ATT_CHUNKS][dh]
    float* ml;  // [slots][hQ][ATT_CHUNKS][2]
};

// grid (ATT_CHUNKS, hKV, slots), 256 threads.  G query heads of one KV head over one position range.
__global__ __launch_bounds__(256) void attn_range_kernel(const float* __restrict__ qhat, const float* __restrict__ kc,
                                                         const float* __restrict__ vc,
                                                         const uint32_t* __restrict__ slot_pos, AttnWs ws, uint32_t hQ,
                                                         uint32_t hKV, uint32_t G, uint32_t tmax)
{
    __shared__ __attribute__((aligned(16))) float s_sc[ATT_GMAX][ATT_TILE];
    __shared__ float s_corr[ATT_GMAX], s_m[ATT_GMAX], s_l[ATT_GMAX];
    const uint32_t c = blockIdx.x, kv = blockIdx.y, rq = blockIdx.z, t = threadIdx.x;
    const uint32_t lane = t & 63u, wave = t >> 6;
    const uint32_t n = slot_position(slot_pos, rq, tmax) + 1u;
    const uint32_t per = (tmax + ATT_CHUNKS - 1) / ATT_CHUNKS;
    const uint32_t p_begin = c * per, p_end = min(n, p_begin + per);
    if (p_begin >= n) return; // the whole workgroup: this range holds no key yet

    // the lane's four dims of every query head, in registers for all tiles
    float4 q[ATT_GMAX];
#pragma unroll
    for (uint32_t h = 0; h < ATT_GMAX; h++)
        q[h] = h < G ? ((const float4*)(qhat + ((size_t)rq * hQ + kv * G + h) * ATT_DH))[lane] : float4{0.f, 0.f, 0.f, 0.f};
    if (t < ATT_GMAX) { s_m[t] = ATT_FLOOR; s_l[t] = 0.f; }
    const float qs = 1.f / sqrtf((float)ATT_DH);
    const float* kbase = kc + ((size_t)rq * hKV + kv) * tmax * ATT_DH;
    const float* vbase = vc + ((size_t)rq * hKV + kv) * tmax * ATT_DH;
    float acc[ATT_GMAX];
#pragma unroll
    for (uint32_t h = 0; h < ATT_GMAX; h++) acc[h] = 0.f;
    __syncthreads();

    for (uint32_t p0 = p_begin; p0 < p_end; p0 += ATT_TILE) {
        const uint32_t ts = min(ATT_TILE, p_end - p0);
        // scores: a wave takes every fourth position of the tile; one coalesced 1 KB row per position
        for (uint32_t i = wave; i < ts; i += 4) {
            const float4 k4 = ((const float4*)(kbase + (size_t)(p0 + i) * ATT_DH))[lane];
#pragma unroll
            for (uint32_t h = 0; h < ATT_GMAX; h++) {
                if (h < G) { // uniform
                    const float d = wave_sum((q[h].x * k4.x + q[h].y * k4.y) + (q[h].z * k4.z + q[h].w * k4.w));
                    if (lane == 0) s_sc[h][i] = d * qs;
                }
            }
        }
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
        // weighted value rows: thread t owns dim t of every head's accumulator
#pragma unroll
        for (uint32_t h = 0; h < ATT_GMAX; h++) acc[h] *= h < G ? s_corr[h] : 0.f;
        for (uint32_t j = 0; j < ts; j++) {
            const float vv = vbase[(size_t)(p0 + j) * ATT_DH + t];
#pragma unroll
            for (uint32_t h = 0; h < ATT_GMAX; h++)
                if (h < G) acc[h] += s_sc[h][j] * vv;
        }
        __syncthreads(); // the next tile overwrites the scores
    }
    for (uint32_t h = 0; h < G; h++) {
        const size_t slot = ((size_t)rq * hQ + kv * G + h) * ATT_CHUNKS + c;
        ws.acc[slot * ATT_DH + t] = acc[h];
        if (t == 0) { ws.ml[2 * slot] = s_m[h]; ws.ml[2 * slot + 1] = s_l[h]; }
    }
}

// grid (hQ, slots), 256 threads: folds the ranges of one query head in range order, divides by the
// sum and applies the output gate sigmoid(qfull[head][dh + t]).
__global__ __launch_bounds__(256) void attn_fold_kernel(AttnWs ws, const float* __restrict__ qfull,
                                                        const uint32_t* __restrict__ slot_pos, float* __restrict__ att,
                                                        uint32_t hQ, uint32_t tmax)
{
    const uint32_t h = blockIdx.x, rq = blockIdx.y, t = threadIdx.x;
    const uint32_t n = slot_position(slot_pos, rq, tmax) + 1u;
    const uint32_t per = (tmax + ATT_CHUNKS - 1) / ATT_CHUNKS;
    const uint32_t n_ranges = min(ATT_CHUNKS, (n + per - 1) / per);
    const size_t base = ((size_t)rq * hQ + h) * ATT_CHUNKS;
    float m = ATT_FLOOR;
    for (uint32_t c = 0; c < n_ranges; c++) m = fmaxf(m, ws.ml[2 * (base + c)]);
    float l = 0.f, o = 0.f;
    for (uint32_t c = 0; c < n_ranges; c++) {
        const float f = expf(ws.ml[2 * (base + c)] - m);
        l += ws.ml[2 * (base + c) + 1] * f;
        o += ws.acc[(base + c) * ATT_DH + t] * f;
    }
    const float g = qfull[((size_t)rq * hQ + h) * 2 * ATT_DH + ATT_DH + t];
    att[((size_t)rq * hQ + h) * ATT_DH + t] = (o / l) * (1.f / (1.f + expf(-g)));
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

int qkk_attn_prep(const float* qfull, const float* kin, const float* vin, const float* q_norm_w, const float* k_norm_w,
                  const float* rope, const uint32_t* slot_pos, float* qhat, float* k_cache, float* v_cache,
                  uint32_t n_slots, uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t n_rot, uint32_t tmax, float eps,
                  void* stream)
{
    if (!qfull || !kin || !vin || !q_norm_w || !k_norm_w || !rope || !slot_pos || !qhat || !k_cache || !v_cache)
        return fail(QKK_EINVAL, "qkk_attn_prep: null pointer");
    if (int rc = check_shape("qkk_attn_prep", n_slots, hQ, hKV, dh, tmax)) return rc;
    if (n_rot < 2 || n_rot % 2 || n_rot > dh) return fail(QKK_ESHAPE, "qkk_attn_prep: n_rot %u must be even, 2..%u", n_rot, dh);
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_attn_prep: eps must be non-negative");
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(attn_prep_kernel, dim3(hQ + 2 * hKV, n_slots), dim3(256), 0, as_stream(stream), qfull, kin, vin,
                       q_norm_w, k_norm_w, rope, slot_pos, qhat, k_cache, v_cache, hQ, hKV, n_rot, tmax, eps);
    return check_launch("qkk_attn_prep");
}

size_t qkk_attn_workspace_bytes(uint32_t n_slots, uint32_t hQ, uint32_t dh)
{
    if (!n_slots || !hQ || !dh) return 0;
    return (size_t)n_slots * hQ * ATT_CHUNKS * ((size_t)dh + 2) * sizeof(float) + 256;
}

int qkk_attn_decode(const float* qhat, const float* k_cache, const float* v_cache, const float* qfull,
                    const uint32_t* slot_pos, float* att, void* workspace, size_t workspace_bytes, uint32_t n_slots,
                    uint32_t hQ, uint32_t hKV, uint32_t dh, uint32_t tmax, void* stream)
{
    if (!qhat || !k_cache || !v_cache || !qfull || !slot_pos || !att || !workspace)
        return fail(QKK_EINVAL, "qkk_attn_decode: null pointer");
    if (int rc = check_shape("qkk_attn_decode", n_slots, hQ, hKV, dh, tmax)) return rc;
    if (!aligned16(qhat) || !aligned16(k_cache) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return fail(QKK_EINVAL, "qkk_attn_decode: qhat and k_cache must be 16-byte, workspace 256-byte aligned");
    if (workspace_bytes < qkk_attn_workspace_bytes(n_slots, hQ, dh))
        return fail(QKK_EWORKSPACE, "qkk_attn_decode: workspace %zu < %zu bytes", workspace_bytes,
                    qkk_attn_workspace_bytes(n_slots, hQ, dh));
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    AttnWs ws;
    ws.acc = (float*)workspace;
    ws.ml = ws.acc + (size_t)n_slots * hQ * ATT_CHUNKS * ATT_DH;
    hipLaunchKernelGGL(attn_range_kernel, dim3(ATT_CHUNKS, hKV, n_slots), dim3(256), 0, st, qhat, k_cache, v_cache,
                       slot_pos, ws, hQ, hKV, hQ / hKV, tmax);
    hipLaunchKernelGGL(attn_fold_kernel, dim3(hQ, n_slots), dim3(256), 0, st, ws, qfull, slot_pos, att, hQ, tmax);
    return check_launch("qkk_attn_decode");
}

} // extern "C"
