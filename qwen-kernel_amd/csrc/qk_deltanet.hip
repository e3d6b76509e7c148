// qk_deltanet.hip -- the gated-DeltaNet mixer's decode step (reference shaders/dn_ab.comp:20-50,
// dn_convn.comp:20-54, dn_step_gate.comp:26-81 = dn_step.comp + dn_gate.comp; host
// src/main.cpp:4200-4244; CPU mirror src/main.cpp:1704-1768).  Per slot and layer:
//   ab    g[h] = a[h] * softplus(alpha_w[h] . x + dt_bias[h]),  beta[h] = sigmoid(beta_w[h] . x)
//   conv  depthwise causal conv over the last 4 inputs of every q/k/v channel + SiLU, the 3-deep
//         input window shifted; q and k heads (dS channels each) scaled to unit length
//   step  per value head h (key/query head kh = h / kdiv, or h % hK when kdiv = 0), state S [dS x dS]:
//           sk_j = exp(g) * sum_i S[j][i] k_i;   d_j = beta * (v_j - sk_j)
//           S[j][i] <- S[j][i] * exp(g) + k_i * d_j;   o_j = sum_i S[j][i] q_i / sqrt(dS)
//         then att[h][j] = o_j / sqrt(mean_j o_j^2 + eps) * norm_w[j] * silu(z[h][j])
// The step is bound by the state: dS*dS*4 bytes read and written per head (2 MiB each way per slot
// at 32 heads of 128).  The state is kept COLUMN-major in memory -- element (row j, column i) at
// [i][j] -- so that the 64 lanes of a wave read 64 consecutive floats for every i (row-major, as in
// the reference, every lane would touch a cache line of its own per request).
#include "qk_device.h"
#include "qk_host.h"

namespace qk {

constexpr uint32_t DN_DS = 128; // state size = channels per head = threads per head

// Sum over the two waves of a 128-thread workgroup, in wave order; every thread gets the same bits.
__device__ __forceinline__ float block_sum2(float v, float* s_red)
{
    const float w = wave_sum(v);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = w;
    __syncthreads();
    return s_red[0] + s_red[1];
}

// grid (ceil(2*hV / 4), slots), 256 threads: one wave per output (h < hV: g, else beta), n = 256*NCH.
template <int NCH>
__global__ __launch_bounds__(256) void dn_ab_kernel(const float* __restrict__ x, const float* __restrict__ alpha_w,
                                                    const float* __restrict__ beta_w, const float* __restrict__ dt_bias,
                                                    const float* __restrict__ a_vec, float* __restrict__ gb, uint32_t hV)
{
    const uint32_t lane = threadIdx.x & 63u, w = blockIdx.x * 4 + (threadIdx.x >> 6), rq = blockIdx.y;
    if (w >= 2 * hV) return; // the whole wave
    const bool is_beta = w >= hV;
    const uint32_t h = is_beta ? w - hV : w;
    const float4* row = (const float4*)((is_beta ? beta_w : alpha_w) + (size_t)h * 256 * NCH);
    const float4* xv = (const float4*)(x + (size_t)rq * 256 * NCH);
    float4 a[NCH], b[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) a[i] = row[lane + 64 * i];
#pragma unroll
    for (int i = 0; i < NCH; i++) b[i] = xv[lane + 64 * i];
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        s0 += a[i].x * b[i].x + a[i].y * b[i].y;
        s1 += a[i].z * b[i].z + a[i].w * b[i].w;
    }
    const float d = wave_sum(s0 + s1);
    if (lane == 0) {
        if (is_beta) {
            gb[(size_t)rq * 2 * hV + hV + h] = 1.f / (1.f + expf(-d));
        } else {
            const float v = d + dt_bias[h];
            gb[(size_t)rq * 2 * hV + h] = a_vec[h] * (v > 20.f ? v : log1pf(expf(v)));
        }
    }
}

// grid (channels / dS, slots), 128 threads: one head of dS channels.
__global__ __launch_bounds__(128) void dn_conv_kernel(float* __restrict__ st, const float* __restrict__ qkv,
                                                      const float* __restrict__ ker, float* __restrict__ out,
                                                      uint32_t channels, uint32_t qk_channels, float eps)
{
    __shared__ float s_red[2];
    const uint32_t ch = blockIdx.x * DN_DS + threadIdx.x, rq = blockIdx.y;
    float* s = st + ((size_t)rq * channels + ch) * 3;
    const float s0 = s[0], s1 = s[1], s2 = s[2], xin = qkv[(size_t)rq * channels + ch];
    const float4 k = ((const float4*)ker)[ch];
    const float c = s0 * k.x + s1 * k.y + s2 * k.z + xin * k.w;
    float v = c / (1.f + expf(-c));
    s[0] = s1; s[1] = s2; s[2] = xin;
    if (blockIdx.x * DN_DS < qk_channels) // a q or k head (uniform): unit length
        v *= 1.f / fmaxf(sqrtf(block_sum2(v * v, s_red)), eps);
    out[(size_t)rq * channels + ch] = v;
}

// dn_ab and dn_conv in one launch for a decode step (neither needs the other's result; two launches
// of 3-5 us each are mostly launch ramp): grid (channels / dS + hV, slots), 128 threads.  Workgroups
// below channels / dS run the conv of one head exactly as dn_conv_kernel; the others form two outputs
// of dn_ab each (one per wave: g of head b and beta of head b), exactly as dn_ab_kernel.
// NORM: x is the residual row and its RMS norm (weights nw) is applied on the way in -- a wave holds
// the whole row, so the mean square is one cross-lane sum and the two dot products are scaled by it.
template <int NCH, bool NORM = false>
__global__ __launch_bounds__(128) void dn_ab_conv_kernel(float* __restrict__ st, const float* __restrict__ qkv,
                                                         const float* __restrict__ ker, float* __restrict__ out,
                                                         uint32_t channels, uint32_t qk_channels, float eps,
                                                         const float* __restrict__ x, const float* __restrict__ alpha_w,
                                                         const float* __restrict__ beta_w, const float* __restrict__ dt_bias,
                                                         const float* __restrict__ a_vec, float* __restrict__ gb, uint32_t hV,
                                                         const float* __restrict__ nw, float norm_eps)
{
    __shared__ float s_red[2];
    const uint32_t rq = blockIdx.y, conv_blocks = channels / DN_DS;
    if (blockIdx.x < conv_blocks) { // uniform per workgroup
        const uint32_t ch = blockIdx.x * DN_DS + threadIdx.x;
        float* s = st + ((size_t)rq * channels + ch) * 3;
        const float s0 = s[0], s1 = s[1], s2 = s[2], xin = qkv[(size_t)rq * channels + ch];
        const float4 k = ((const float4*)ker)[ch];
        const float c = s0 * k.x + s1 * k.y + s2 * k.z + xin * k.w;
        float v = c / (1.f + expf(-c));
        s[0] = s1; s[1] = s2; s[2] = xin;
        if (blockIdx.x * DN_DS < qk_channels) v *= 1.f / fmaxf(sqrtf(block_sum2(v * v, s_red)), eps);
        out[(size_t)rq * channels + ch] = v;
        return;
    }
    const uint32_t lane = threadIdx.x & 63u, h = blockIdx.x - conv_blocks;
    const bool is_beta = threadIdx.x >= 64; // wave 0: g, wave 1: beta
    const float4* row = (const float4*)((is_beta ? beta_w : alpha_w) + (size_t)h * 256 * NCH);
    const float4* xv = (const float4*)(x + (size_t)rq * 256 * NCH);
    float4 a[NCH], b[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) a[i] = row[lane + 64 * i];
#pragma unroll
    for (int i = 0; i < NCH; i++) b[i] = xv[lane + 64 * i];
    float scale = 1.f;
    if constexpr (NORM) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const float4 g = ((const float4*)nw)[lane + 64 * i];
            ss += (b[i].x * b[i].x + b[i].y * b[i].y) + (b[i].z * b[i].z + b[i].w * b[i].w);
            b[i] = float4{b[i].x * g.x, b[i].y * g.y, b[i].z * g.z, b[i].w * g.w};
        }
        scale = 1.f / sqrtf(wave_sum(ss) / (float)(256 * NCH) + norm_eps);
    }
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        p0 += a[i].x * b[i].x + a[i].y * b[i].y;
        p1 += a[i].z * b[i].z + a[i].w * b[i].w;
    }
    const float d = wave_sum(p0 + p1) * scale;
    if (lane == 0) {
        if (is_beta) {
            gb[(size_t)rq * 2 * hV + hV + h] = 1.f / (1.f + expf(-d));
        } else {
            const float v = d + dt_bias[h];
            gb[(size_t)rq * 2 * hV + h] = a_vec[h] * (v > 20.f ? v : log1pf(expf(v)));
        }
    }
}

// The step: grid (hV, slots), 128 * DN_PARTS threads.  A row's columns are cut into DN_PARTS parts:
// thread (row j = t % 128, part c = t / 128) keeps dS / DN_PARTS state values -- one round of loads --
// and the two sums over columns are finished through LDS (a wave holds one part of 64 consecutive
// rows, so every load and store stays a run of consecutive floats).  A thread per whole row (dS
// loads each, 128 threads per head) took 7.9 us for one slot against 5.6 us, 17.2 / 16.7 us for 16.
constexpr uint32_t DN_PARTS = 8, DN_PC = DN_DS / DN_PARTS;

__global__ __launch_bounds__(DN_DS* DN_PARTS) void dn_step_kernel(const float* __restrict__ conv,
                                                                         const float* __restrict__ gb,
                                                                         float* __restrict__ state,
                                                                         const float* __restrict__ norm_w,
                                                                         const float* __restrict__ z, float* __restrict__ att,
                                                                         uint32_t hK, uint32_t hV, uint32_t kdiv, float eps)
{
    __shared__ float s_q[DN_DS], s_k[DN_DS];
    __shared__ float s_part[2][DN_PARTS][DN_DS];
    __shared__ float s_red[2];
    const uint32_t h = blockIdx.x, rq = blockIdx.y, j = threadIdx.x % DN_DS, c = threadIdx.x / DN_DS;
    const uint32_t kh = kdiv ? min(h / kdiv, hK - 1) : h % hK;
    const float* cv = conv + (size_t)rq * (2 * hK + hV) * DN_DS;
    float* S = state + ((size_t)rq * hV + h) * DN_DS * DN_DS + (size_t)c * DN_PC * DN_DS + j; // (row j, column 16c + i) at [i * dS]
    float s[DN_PC];
#pragma unroll
    for (uint32_t i = 0; i < DN_PC; i++) s[i] = S[(size_t)i * DN_DS];
    if (c == 0) s_q[j] = cv[(size_t)kh * DN_DS + j] * (1.f / sqrtf((float)DN_DS));
    if (c == 1) s_k[j] = cv[(size_t)(hK + kh) * DN_DS + j];
    const float vj = cv[(size_t)(2 * hK + h) * DN_DS + j];
    const float decay = expf(gb[(size_t)rq * 2 * hV + h]), beta = gb[(size_t)rq * 2 * hV + hV + h];
    const float zv = z[((size_t)rq * hV + h) * DN_DS + j], nw = norm_w[j];
    __syncthreads();
    float kk[DN_PC], ps = 0.f;
#pragma unroll
    for (uint32_t i = 0; i < DN_PC; i++) {
        kk[i] = s_k[c * DN_PC + i];
        ps += s[i] * kk[i];
    }
    s_part[0][c][j] = ps;
    __syncthreads();
    float sk = 0.f;
#pragma unroll
    for (uint32_t p = 0; p < DN_PARTS; p++) sk += s_part[0][p][j];
    const float dj = beta * (vj - sk * decay);
    float po = 0.f;
#pragma unroll
    for (uint32_t i = 0; i < DN_PC; i++) {
        const float sn = s[i] * decay + kk[i] * dj;
        S[(size_t)i * DN_DS] = sn;
        po += sn * s_q[c * DN_PC + i];
    }
    s_part[1][c][j] = po;
    __syncthreads();
    if (c == 0) { // waves 0 and 1: the head's 128 rows
        float oj = 0.f;
#pragma unroll
        for (uint32_t p = 0; p < DN_PARTS; p++) oj += s_part[1][p][j];
        const float w = wave_sum(oj * oj);
        if ((j & 63u) == 0) s_red[j >> 6] = w;
        s_part[0][0][j] = oj;
    }
    __syncthreads();
    if (c == 0) {
        const float oj = s_part[0][0][j];
        const float scale = 1.f / sqrtf((s_red[0] + s_red[1]) / (float)DN_DS + eps);
        att[((size_t)rq * hV + h) * DN_DS + j] = oj * scale * nw * (zv / (1.f + expf(-zv)));
    }
}

// ---- the whole decode step of the mixer in ONE launch --------------------------------------------
// ab, conv and step for the value heads of one key head per workgroup: grid (hK, slots), 1024 threads,
// for shapes with two value heads per key head (the reference's 32 on 16).  The q / k conv window of a
// key head is read by both of its value heads but may be shifted once only, and not before both have
// read it -- inside one workgroup that is a barrier, across workgroups it would be a race: hence the
// key head as the unit.  Same arithmetic in the same order as dn_ab_conv_kernel followed by
// dn_step_kernel (the results are bit for bit theirs); what is saved is a launch and the round trip
// of conv and gb through memory.
//   threads    0..127 q channels, 128..255 k channels, 256..383 v of head A, 384..511 v of head B: conv +
//              SiLU + window shift; q and k scaled to unit length (two waves each: one LDS exchange)
//   waves 8..11 one dot product each: alpha . x and beta . x of head A and of head B
//   then every thread (row j = t % 128, part c = t / 128) holds dS / 8 state values of BOTH heads and
//   runs the delta rule on them with the shared q and k; the column sums of both heads share the
//   barriers.
// NORM as in dn_ab_conv_kernel.
template <int NCH, bool NORM>
__global__ __launch_bounds__(DN_DS* DN_PARTS) void dn_fused_step_kernel(
    float* __restrict__ win, const float* __restrict__ qkv, const float* __restrict__ ker, const float* __restrict__ x,
    const float* __restrict__ nw, float norm_eps, const float* __restrict__ alpha_w, const float* __restrict__ beta_w,
    const float* __restrict__ dt_bias, const float* __restrict__ a_vec, float* __restrict__ state,
    const float* __restrict__ norm_w, const float* __restrict__ z, float* __restrict__ att, uint32_t hK, uint32_t hV,
    uint32_t kdiv, float eps)
{
    __shared__ float s_q[DN_DS], s_k[DN_DS], s_v[2][DN_DS];
    __shared__ float s_part[2][2][DN_PARTS][DN_DS]; // [head][k or q sums][part][row]
    __shared__ float s_red[2][2], s_qk[4], s_gb[4]; // q/k squares per wave; decay A, decay B, beta A, beta B
    const uint32_t kh = blockIdx.x, rq = blockIdx.y, t = threadIdx.x, j = t % DN_DS, c = t / DN_DS, lane = t & 63u;
    const uint32_t channels = (2 * hK + hV) * DN_DS;
    const uint32_t hd[2] = {kdiv ? kh * kdiv : kh, kdiv ? kh * kdiv + 1 : kh + hK}; // the two value heads of key head kh

    // the state of both heads: requested before anything else -- except by the four waves that form the dot
    // products, whose operands need the registers first (they request it when those are done)
    float s[2][DN_PC];
    float* S[2];
    const bool dots = c == 4 || c == 5; // uniform per wave
#pragma unroll
    for (int a = 0; a < 2; a++) S[a] = state + ((size_t)rq * hV + hd[a]) * DN_DS * DN_DS + (size_t)c * DN_PC * DN_DS + j;
    if (!dots) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (uint32_t i = 0; i < DN_PC; i++) s[a][i] = S[a][(size_t)i * DN_DS];
    }
    const float zv[2] = {z[((size_t)rq * hV + hd[0]) * DN_DS + j], z[((size_t)rq * hV + hd[1]) * DN_DS + j]};
    const float nwj = norm_w[j];

    if (c < 4) { // conv of one channel: q, k, v of head A, v of head B
        const uint32_t ch = (c == 0 ? kh : c == 1 ? hK + kh : 2 * hK + hd[c - 2]) * DN_DS + j;
        float* w = win + ((size_t)rq * channels + ch) * 3;
        const float w0 = w[0], w1 = w[1], w2 = w[2], xin = qkv[(size_t)rq * channels + ch];
        const float4 kk = ((const float4*)ker)[ch];
        const float cv = w0 * kk.x + w1 * kk.y + w2 * kk.z + xin * kk.w;
        const float v = cv / (1.f + expf(-cv));
        w[0] = w1; w[1] = w2; w[2] = xin;
        if (c < 2) { // a q or k head: its squares, wave by wave
            const float sq = wave_sum(v * v);
            if (lane == 0) s_qk[t >> 6] = sq;
            (c == 0 ? s_q : s_k)[j] = v;
        } else {
            s_v[c - 2][j] = v;
        }
    } else if (c < 6) { // waves 8..11: alpha A, alpha B, beta A, beta B
        const uint32_t wv = (t >> 6) - 8, a = wv & 1u;
        const bool is_beta = wv >= 2;
        const float4* row = (const float4*)((is_beta ? beta_w : alpha_w) + (size_t)hd[a] * 256 * NCH);
        const float4* xv = (const float4*)(x + (size_t)rq * 256 * NCH);
        float4 ra[NCH], rb[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) ra[i] = row[lane + 64 * i];
#pragma unroll
        for (int i = 0; i < NCH; i++) rb[i] = xv[lane + 64 * i];
        float scale = 1.f;
        if constexpr (NORM) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const float4 g = ((const float4*)nw)[lane + 64 * i];
                ss += (rb[i].x * rb[i].x + rb[i].y * rb[i].y) + (rb[i].z * rb[i].z + rb[i].w * rb[i].w);
                rb[i] = float4{rb[i].x * g.x, rb[i].y * g.y, rb[i].z * g.z, rb[i].w * g.w};
            }
            scale = 1.f / sqrtf(wave_sum(ss) / (float)(256 * NCH) + norm_eps);
        }
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            p0 += ra[i].x * rb[i].x + ra[i].y * rb[i].y;
            p1 += ra[i].z * rb[i].z + ra[i].w * rb[i].w;
        }
        const float d = wave_sum(p0 + p1) * scale;
        if (lane == 0) {
            if (is_beta) {
                s_gb[2 + a] = 1.f / (1.f + expf(-d));
            } else {
                const float v = d + dt_bias[hd[a]];
                s_gb[a] = expf(a_vec[hd[a]] * (v > 20.f ? v : log1pf(expf(v))));
            }
        }
#pragma unroll
        for (int a2 = 0; a2 < 2; a2++)
#pragma unroll
            for (uint32_t i = 0; i < DN_PC; i++) s[a2][i] = S[a2][(size_t)i * DN_DS];
    }
    __syncthreads();
    // unit length for q and k (as block_sum2 in dn_conv_kernel: the two waves' sums in wave order), q also / sqrt(dS)
    if (c == 0) s_q[j] = s_q[j] * (1.f / fmaxf(sqrtf(s_qk[0] + s_qk[1]), eps)) * (1.f / sqrtf((float)DN_DS));
    if (c == 1) s_k[j] = s_k[j] * (1.f / fmaxf(sqrtf(s_qk[2] + s_qk[3]), eps));
    __syncthreads();

    float kk[DN_PC];
#pragma unroll
    for (uint32_t i = 0; i < DN_PC; i++) kk[i] = s_k[c * DN_PC + i];
#pragma unroll
    for (int a = 0; a < 2; a++) {
        float ps = 0.f;
#pragma unroll
        for (uint32_t i = 0; i < DN_PC; i++) ps += s[a][i] * kk[i];
        s_part[a][0][c][j] = ps;
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < 2; a++) {
        float sk = 0.f;
#pragma unroll
        for (uint32_t p = 0; p < DN_PARTS; p++) sk += s_part[a][0][p][j];
        const float decay = s_gb[a], beta = s_gb[2 + a];
        const float dj = beta * (s_v[a][j] - sk * decay);
        float po = 0.f;
#pragma unroll
        for (uint32_t i = 0; i < DN_PC; i++) {
            const float sn = s[a][i] * decay + kk[i] * dj;
            S[a][(size_t)i * DN_DS] = sn;
            po += sn * s_q[c * DN_PC + i];
        }
        s_part[a][1][c][j] = po;
    }
    __syncthreads();
    if (c < 2) { // parts 0 and 1: the 128 rows of head A and of head B
        float oj = 0.f;
#pragma unroll
        for (uint32_t p = 0; p < DN_PARTS; p++) oj += s_part[c][1][p][j];
        const float w = wave_sum(oj * oj);
        if (lane == 0) s_red[c][(t >> 6) & 1u] = w;
        s_part[c][0][0][j] = oj;
    }
    __syncthreads();
    if (c < 2) {
        const float oj = s_part[c][0][0][j];
        const float scale = 1.f / sqrtf((s_red[c][0] + s_red[c][1]) / (float)DN_DS + eps);
        att[((size_t)rq * hV + hd[c]) * DN_DS + j] = oj * scale * nwj * (zv[c] / (1.f + expf(-zv[c])));
    }
}

// The same two steps over n_pos consecutive positions of ONE slot (reference
// shaders/dn_conv_batch.comp, dn_step_batch.comp + dn_gate_batch.comp): rows t of qkv / conv / gb /
// z / att are positions; the window and the state are read once and written once.

// The conv is a 4-tap filter over the inputs, not a recurrence: position t needs the inputs t-3..t,
// the first three positions taking the missing ones from the window.  grid (channels / dS, positions),
// 128 threads; the window itself is moved on by dn_window_seq_kernel afterwards.
__global__ __launch_bounds__(128) void dn_conv_seq_kernel(const float* __restrict__ st, const float* __restrict__ qkv,
                                                          const float* __restrict__ ker, float* __restrict__ out,
                                                          uint32_t channels, uint32_t qk_channels, float eps)
{
    __shared__ float s_red[2];
    const uint32_t ch = blockIdx.x * DN_DS + threadIdx.x, t = blockIdx.y;
    auto input = [&](int u) { return u >= 0 ? qkv[(size_t)u * channels + ch] : st[(size_t)ch * 3 + (3 + u)]; };
    const float s0 = input((int)t - 3), s1 = input((int)t - 2), s2 = input((int)t - 1), xin = input((int)t);
    const float4 k = ((const float4*)ker)[ch];
    const float c = s0 * k.x + s1 * k.y + s2 * k.z + xin * k.w;
    float v = c / (1.f + expf(-c));
    if (blockIdx.x * DN_DS < qk_channels) // a q or k head (uniform): unit length
        v *= 1.f / fmaxf(sqrtf(block_sum2(v * v, s_red)), eps);
    out[(size_t)t * channels + ch] = v;
}

// grid (channels / dS), 128 threads: the window after n_pos positions = the last three inputs.
__global__ __launch_bounds__(128) void dn_window_seq_kernel(float* __restrict__ st, const float* __restrict__ qkv,
                                                            uint32_t channels, uint32_t n_pos)
{
    const uint32_t ch = blockIdx.x * DN_DS + threadIdx.x;
    float* s = st + (size_t)ch * 3;
    auto input = [&](int u) { return u >= 0 ? qkv[(size_t)u * channels + ch] : s[3 + u]; };
    const float a = input((int)n_pos - 3), b = input((int)n_pos - 2), c = input((int)n_pos - 1);
    s[0] = a; s[1] = b; s[2] = c;
}

// The delta rule over the positions is one serial chain per state row, and a head has only dS rows:
// a workgroup per head would leave most of the chip idle and spend ~3 dS multiply-adds per thread
// and position.  So a head is cut into SEQ_RB-row blocks (hV * dS / SEQ_RB workgroups) and every row
// into SEQ_NQ parts of its columns: thread (row r, part c) keeps dS/SEQ_NQ state values and the two
// sums over columns are finished across the SEQ_NQ neighbouring lanes.  q, k, v and the gates of
// SEQ_CH positions at a time are staged in LDS (double-buffered; the next chunk's global loads are
// in flight while the current one is worked on), one barrier per chunk.  The head-wide norm and the
// output gate need all rows of a head and run as a second kernel over (head, position).
constexpr uint32_t SEQ_NQ = 16;              // lanes per state row
constexpr uint32_t SEQ_RB = 128 / SEQ_NQ;    // state rows per workgroup of 128 threads
constexpr uint32_t SEQ_CH = 16;              // positions per staged chunk
constexpr uint32_t SEQ_QS = DN_DS / SEQ_NQ;  // columns per part
constexpr uint32_t SEQ_PAD = SEQ_QS + 4;     // part stride in LDS: the parts' float4 reads hit distinct banks
constexpr uint32_t SEQ_TOTAL = SEQ_CH * (2 * DN_DS + SEQ_RB) / 4; // float4 loads per chunk
constexpr uint32_t SEQ_ITEMS = (SEQ_TOTAL + 127) / 128;           // per thread
static_assert(2 * SEQ_CH <= 128 && (SEQ_NQ == 4 || SEQ_NQ == 8 || SEQ_NQ == 16), "chunk staging");

struct SeqChunk {
    float q[SEQ_CH][SEQ_NQ * SEQ_PAD];
    float k[SEQ_CH][SEQ_NQ * SEQ_PAD];
    float v[SEQ_CH][SEQ_RB];
    float g[SEQ_CH][2]; // decay = exp(log decay), write strength
};

// grid (hV * dS / SEQ_RB), 128 threads.  att receives the raw o_j; dn_gate_seq_kernel finishes it.
__global__ __launch_bounds__(128) void dn_step_seq_kernel(const float* __restrict__ conv, const float* __restrict__ gb,
                                                          float* __restrict__ state, float* __restrict__ att, uint32_t hK,
                                                          uint32_t hV, uint32_t kdiv, uint32_t n_pos)
{
    __shared__ __attribute__((aligned(16))) SeqChunk s_c[2];
    constexpr uint32_t BPH = DN_DS / SEQ_RB, PER_POS = (2 * DN_DS + SEQ_RB) / 4;
    const uint32_t h = blockIdx.x / BPH, rb = blockIdx.x % BPH, tid = threadIdx.x;
    const uint32_t r = tid / SEQ_NQ, c = tid % SEQ_NQ, row = rb * SEQ_RB + r;
    const uint32_t kh = kdiv ? min(h / kdiv, hK - 1) : h % hK;
    const size_t cstride = (size_t)(2 * hK + hV) * DN_DS;
    const float q_scale = 1.f / sqrtf((float)DN_DS);
    float* S = state + (size_t)h * DN_DS * DN_DS; // column-major: (row, column i) at [i][row]
    float s[SEQ_QS];
#pragma unroll
    for (uint32_t i = 0; i < SEQ_QS; i++) s[i] = S[(size_t)(c * SEQ_QS + i) * DN_DS + row];

    float4 pre[SEQ_ITEMS];
    float pre_g = 0.f;
    // item x of a chunk: position x / PER_POS; word w = x % PER_POS: float4 w of q, w - 32 of k, w - 64 of the block's v
    auto fetch = [&](uint32_t t0) {
#pragma unroll
        for (uint32_t it = 0; it < SEQ_ITEMS; it++) {
            const uint32_t x = min(tid + 128 * it, SEQ_TOTAL - 1), p = x / PER_POS, w = x % PER_POS;
            const uint32_t t = min(t0 + p, n_pos - 1); // positions beyond the end repeat the last one, unused
            const float* cv = conv + (size_t)t * cstride;
            const float* src = w < DN_DS / 4       ? cv + (size_t)kh * DN_DS + 4 * w
                               : w < 2 * DN_DS / 4 ? cv + (size_t)(hK + kh) * DN_DS + 4 * (w - DN_DS / 4)
                                                   : cv + (size_t)(2 * hK + h) * DN_DS + rb * SEQ_RB + 4 * (w - 2 * DN_DS / 4);
            pre[it] = *(const float4*)src;
        }
        if (tid < 2 * SEQ_CH) {
            const uint32_t t = min(t0 + (tid >> 1), n_pos - 1);
            pre_g = gb[(size_t)t * 2 * hV + (tid & 1u) * hV + h];
        }
    };
    auto stage = [&](uint32_t b) {
#pragma unroll
        for (uint32_t it = 0; it < SEQ_ITEMS; it++) {
            const uint32_t x = tid + 128 * it, p = x / PER_POS, w = x % PER_POS;
            float4 v = pre[it];
            if (x >= SEQ_TOTAL) {
            } else if (w < DN_DS / 4) {
                v.x *= q_scale; v.y *= q_scale; v.z *= q_scale; v.w *= q_scale;
                *(float4*)&s_c[b].q[p][(4 * w / SEQ_QS) * SEQ_PAD + 4 * w % SEQ_QS] = v;
            } else if (w < 2 * DN_DS / 4) {
                const uint32_t e = 4 * (w - DN_DS / 4);
                *(float4*)&s_c[b].k[p][(e / SEQ_QS) * SEQ_PAD + e % SEQ_QS] = v;
            } else {
                *(float4*)&s_c[b].v[p][4 * (w - 2 * DN_DS / 4)] = v;
            }
        }
        if (tid < 2 * SEQ_CH) s_c[b].g[tid >> 1][tid & 1u] = (tid & 1u) ? pre_g : expf(pre_g);
    };

    fetch(0);
    stage(0);
    __syncthreads();
    for (uint32_t t0 = 0; t0 < n_pos; t0 += SEQ_CH) {
        const uint32_t b = (t0 / SEQ_CH) & 1u;
        const bool more = t0 + SEQ_CH < n_pos;
        if (more) fetch(t0 + SEQ_CH);
        const uint32_t np = min(SEQ_CH, n_pos - t0);
        auto position = [&](uint32_t p) {
            const float4* k4 = (const float4*)&s_c[b].k[p][c * SEQ_PAD];
            const float4* q4 = (const float4*)&s_c[b].q[p][c * SEQ_PAD];
            const float decay = s_c[b].g[p][0], beta = s_c[b].g[p][1], vj = s_c[b].v[p][r];
            float4 kk[SEQ_QS / 4];
            float4 ps = float4{0.f, 0.f, 0.f, 0.f}; // four independent sums: the chain of multiply-adds is the critical path
#pragma unroll
            for (uint32_t i = 0; i < SEQ_QS / 4; i++) {
                kk[i] = k4[i];
                ps.x += s[4 * i] * kk[i].x; ps.y += s[4 * i + 1] * kk[i].y;
                ps.z += s[4 * i + 2] * kk[i].z; ps.w += s[4 * i + 3] * kk[i].w;
            }
            float sk = (ps.x + ps.y) + (ps.z + ps.w);
            sk += dpp_f<DPP_XOR1>(sk);
            sk += dpp_f<DPP_XOR2>(sk);
            if (SEQ_NQ >= 8) sk += dpp_f<DPP_HALF_MIRROR>(sk);
            if (SEQ_NQ >= 16) sk += dpp_f<DPP_MIRROR>(sk);
            const float dj = beta * (vj - sk * decay);
            float4 po = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (uint32_t i = 0; i < SEQ_QS / 4; i++) {
                const float4 qq = q4[i];
                const float a0 = s[4 * i] * decay + kk[i].x * dj, a1 = s[4 * i + 1] * decay + kk[i].y * dj;
                const float a2 = s[4 * i + 2] * decay + kk[i].z * dj, a3 = s[4 * i + 3] * decay + kk[i].w * dj;
                s[4 * i] = a0; s[4 * i + 1] = a1; s[4 * i + 2] = a2; s[4 * i + 3] = a3;
                po.x += a0 * qq.x; po.y += a1 * qq.y; po.z += a2 * qq.z; po.w += a3 * qq.w;
            }
            float oj = (po.x + po.y) + (po.z + po.w);
            oj += dpp_f<DPP_XOR1>(oj);
            oj += dpp_f<DPP_XOR2>(oj);
            if (SEQ_NQ >= 8) oj += dpp_f<DPP_HALF_MIRROR>(oj);
            if (SEQ_NQ >= 16) oj += dpp_f<DPP_MIRROR>(oj);
            if (c == 0) att[((size_t)(t0 + p) * hV + h) * DN_DS + row] = oj;
        };
        if (np == SEQ_CH) { // whole chunk: unrolled, so that the next position's LDS reads can start early
#pragma unroll 4
            for (uint32_t p = 0; p < SEQ_CH; p++) position(p);
        } else {
            for (uint32_t p = 0; p < np; p++) position(p);
        }
        if (more) stage(b ^ 1u);
        __syncthreads();
    }
#pragma unroll
    for (uint32_t i = 0; i < SEQ_QS; i++) S[(size_t)(c * SEQ_QS + i) * DN_DS + row] = s[i];
}

// grid (hV, positions), 128 threads: att <- att / rms(att over the head) * norm_w * silu(z), in place.
__global__ __launch_bounds__(128) void dn_gate_seq_kernel(float* __restrict__ att, const float* __restrict__ norm_w,
                                                          const float* __restrict__ z, uint32_t hV, float eps)
{
    __shared__ float s_red[2];
    const size_t at = ((size_t)blockIdx.y * hV + blockIdx.x) * DN_DS + threadIdx.x;
    const float oj = att[at], zv = z[at], nw = norm_w[threadIdx.x];
    const float scale = 1.f / sqrtf(block_sum2(oj * oj, s_red) / (float)DN_DS + eps);
    att[at] = oj * scale * nw * (zv / (1.f + expf(-zv)));
}

static int check_slots(const char* who, uint32_t n_slots)
{
    if (n_slots < 1 || n_slots > 65535) return fail(QKK_ESHAPE, "%s: %u slots outside 1..65535", who, n_slots);
    return QKK_OK;
}

} // namespace qk

using namespace qk;

extern "C" {

int qkk_dn_ab(const float* x, const float* alpha_w, const float* beta_w, const float* dt_bias, const float* a_vec,
              float* gb, uint32_t n_embd, uint32_t hV, uint32_t n_slots, void* stream)
{
    if (!x || !alpha_w || !beta_w || !dt_bias || !a_vec || !gb) return fail(QKK_EINVAL, "qkk_dn_ab: null pointer");
    if (int rc = check_slots("qkk_dn_ab", n_slots)) return rc;
    if (n_embd != 2048 && n_embd != 4096) return fail(QKK_ESHAPE, "qkk_dn_ab: n_embd %u not supported (2048 or 4096)", n_embd);
    if (hV < 1 || hV > 4096) return fail(QKK_ESHAPE, "qkk_dn_ab: %u heads outside 1..4096", hV);
    if (!aligned16(x) || !aligned16(alpha_w) || !aligned16(beta_w))
        return fail(QKK_EINVAL, "qkk_dn_ab: x and the weight rows must be 16-byte aligned");
    if (int rc = require_device()) return rc;
    const dim3 grid((2 * hV + 3) / 4, n_slots), block(256);
    if (n_embd == 2048)
        hipLaunchKernelGGL(dn_ab_kernel<8>, grid, block, 0, as_stream(stream), x, alpha_w, beta_w, dt_bias, a_vec, gb, hV);
    else
        hipLaunchKernelGGL(dn_ab_kernel<16>, grid, block, 0, as_stream(stream), x, alpha_w, beta_w, dt_bias, a_vec, gb, hV);
    return check_launch("qkk_dn_ab");
}

int qkk_dn_conv(float* conv_state, const float* qkv, const float* ker, float* out, uint32_t channels, uint32_t d_state,
                uint32_t qk_channels, float eps, uint32_t n_slots, void* stream)
{
    if (!conv_state || !qkv || !ker || !out) return fail(QKK_EINVAL, "qkk_dn_conv: null pointer");
    if (int rc = check_slots("qkk_dn_conv", n_slots)) return rc;
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "qkk_dn_conv: state size %u not supported (128)", d_state);
    if (channels < DN_DS || channels % DN_DS || qk_channels % DN_DS || qk_channels > channels || channels > (1u << 24))
        return fail(QKK_ESHAPE, "qkk_dn_conv: %u channels (%u of q and k) must be whole heads of %u", channels, qk_channels,
                    DN_DS);
    if (!aligned16(ker)) return fail(QKK_EINVAL, "qkk_dn_conv: ker must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_conv: eps must be non-negative");
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(dn_conv_kernel, dim3(channels / DN_DS, n_slots), dim3(DN_DS), 0, as_stream(stream), conv_state, qkv,
                       ker, out, channels, qk_channels, eps);
    return check_launch("qkk_dn_conv");
}

static int dn_ab_conv_impl(const float* x, const float* w_norm, float norm_eps, const float* alpha_w, const float* beta_w,
                           const float* dt_bias, const float* a_vec, float* gb, uint32_t n_embd, uint32_t hV,
                           float* conv_state, const float* qkv, const float* ker, float* out, uint32_t channels,
                           uint32_t d_state, uint32_t qk_channels, float eps, uint32_t n_slots, void* stream)
{
    if (!x || !alpha_w || !beta_w || !dt_bias || !a_vec || !gb || !conv_state || !qkv || !ker || !out)
        return fail(QKK_EINVAL, "qkk_dn_ab_conv: null pointer");
    if (int rc = check_slots("qkk_dn_ab_conv", n_slots)) return rc;
    if (n_embd != 2048 && n_embd != 4096)
        return fail(QKK_ESHAPE, "qkk_dn_ab_conv: n_embd %u not supported (2048 or 4096)", n_embd);
    if (hV < 1 || hV > 4096) return fail(QKK_ESHAPE, "qkk_dn_ab_conv: %u heads outside 1..4096", hV);
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "qkk_dn_ab_conv: state size %u not supported (128)", d_state);
    if (channels < DN_DS || channels % DN_DS || qk_channels % DN_DS || qk_channels > channels || channels > (1u << 24))
        return fail(QKK_ESHAPE, "qkk_dn_ab_conv: %u channels (%u of q and k) must be whole heads of %u", channels,
                    qk_channels, DN_DS);
    if (!aligned16(x) || !aligned16(alpha_w) || !aligned16(beta_w) || !aligned16(ker))
        return fail(QKK_EINVAL, "qkk_dn_ab_conv: x, the weight rows and ker must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_ab_conv: eps must be non-negative");
    if (int rc = require_device()) return rc;
    const dim3 grid(channels / DN_DS + hV, n_slots), block(DN_DS);
    if (w_norm) {
        if (n_embd != 2048) return fail(QKK_ESHAPE, "qkk_dn_ab_conv_norm: n_embd %u not supported (2048)", n_embd);
        hipLaunchKernelGGL((dn_ab_conv_kernel<8, true>), grid, block, 0, as_stream(stream), conv_state, qkv, ker, out, channels,
                           qk_channels, eps, x, alpha_w, beta_w, dt_bias, a_vec, gb, hV, w_norm, norm_eps);
    } else if (n_embd == 2048)
        hipLaunchKernelGGL(dn_ab_conv_kernel<8>, grid, block, 0, as_stream(stream), conv_state, qkv, ker, out, channels,
                           qk_channels, eps, x, alpha_w, beta_w, dt_bias, a_vec, gb, hV, (const float*)nullptr, 0.f);
    else
        hipLaunchKernelGGL(dn_ab_conv_kernel<16>, grid, block, 0, as_stream(stream), conv_state, qkv, ker, out, channels,
                           qk_channels, eps, x, alpha_w, beta_w, dt_bias, a_vec, gb, hV, (const float*)nullptr, 0.f);
    return check_launch("qkk_dn_ab_conv");
}

int qkk_dn_ab_conv(const float* x, const float* alpha_w, const float* beta_w, const float* dt_bias, const float* a_vec,
                   float* gb, uint32_t n_embd, uint32_t hV, float* conv_state, const float* qkv, const float* ker, float* out,
                   uint32_t channels, uint32_t d_state, uint32_t qk_channels, float eps, uint32_t n_slots, void* stream)
{
    return dn_ab_conv_impl(x, nullptr, 0.f, alpha_w, beta_w, dt_bias, a_vec, gb, n_embd, hV, conv_state, qkv, ker, out,
                           channels, d_state, qk_channels, eps, n_slots, stream);
}

int qkk_dn_ab_conv_norm(const float* x, const float* w_norm, float norm_eps, const float* alpha_w, const float* beta_w,
                        const float* dt_bias, const float* a_vec, float* gb, uint32_t n_embd, uint32_t hV,
                        float* conv_state, const float* qkv, const float* ker, float* out, uint32_t channels,
                        uint32_t d_state, uint32_t qk_channels, float eps, uint32_t n_slots, void* stream)
{
    if (!w_norm || !aligned16(w_norm)) return fail(QKK_EINVAL, "qkk_dn_ab_conv_norm: w_norm must be a 16-byte aligned pointer");
    if (!(norm_eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_ab_conv_norm: norm_eps must be non-negative");
    return dn_ab_conv_impl(x, w_norm, norm_eps, alpha_w, beta_w, dt_bias, a_vec, gb, n_embd, hV, conv_state, qkv, ker, out,
                           channels, d_state, qk_channels, eps, n_slots, stream);
}

int qkk_dn_conv_seq(float* conv_state, const float* qkv, const float* ker, float* out, uint32_t channels, uint32_t d_state,
                    uint32_t qk_channels, float eps, uint32_t n_pos, void* stream)
{
    if (!conv_state || !qkv || !ker || !out) return fail(QKK_EINVAL, "qkk_dn_conv_seq: null pointer");
    if (n_pos < 1 || n_pos > (1u << 20)) return fail(QKK_ESHAPE, "qkk_dn_conv_seq: %u positions outside 1..2^20", n_pos);
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "qkk_dn_conv_seq: state size %u not supported (128)", d_state);
    if (channels < DN_DS || channels % DN_DS || qk_channels % DN_DS || qk_channels > channels || channels > (1u << 24))
        return fail(QKK_ESHAPE, "qkk_dn_conv_seq: %u channels (%u of q and k) must be whole heads of %u", channels,
                    qk_channels, DN_DS);
    if (!aligned16(ker)) return fail(QKK_EINVAL, "qkk_dn_conv_seq: ker must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_conv_seq: eps must be non-negative");
    if (int rc = require_device()) return rc;
    if (n_pos > 65535) return fail(QKK_ESHAPE, "qkk_dn_conv_seq: %u positions above 65535", n_pos);
    hipLaunchKernelGGL(dn_conv_seq_kernel, dim3(channels / DN_DS, n_pos), dim3(DN_DS), 0, as_stream(stream), conv_state, qkv,
                       ker, out, channels, qk_channels, eps);
    hipLaunchKernelGGL(dn_window_seq_kernel, dim3(channels / DN_DS), dim3(DN_DS), 0, as_stream(stream), conv_state, qkv,
                       channels, n_pos);
    return check_launch("qkk_dn_conv_seq");
}

int qkk_dn_step_seq(const float* conv, const float* gb, float* state, const float* norm_w, const float* z, float* att,
                    uint32_t d_state, uint32_t hK, uint32_t hV, uint32_t kdiv, float eps, uint32_t n_pos, void* stream)
{
    if (!conv || !gb || !state || !norm_w || !z || !att) return fail(QKK_EINVAL, "qkk_dn_step_seq: null pointer");
    if (n_pos < 1 || n_pos > (1u << 20)) return fail(QKK_ESHAPE, "qkk_dn_step_seq: %u positions outside 1..2^20", n_pos);
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "qkk_dn_step_seq: state size %u not supported (128)", d_state);
    if (hK < 1 || hV < 1 || hV > 65535 || hK > 65535) return fail(QKK_ESHAPE, "qkk_dn_step_seq: head counts out of range");
    if (kdiv ? (hV + kdiv - 1) / kdiv > hK : false)
        return fail(QKK_ESHAPE, "qkk_dn_step_seq: %u value heads / %u exceed %u key heads", hV, kdiv, hK);
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_step_seq: eps must be non-negative");
    if (int rc = require_device()) return rc;
    if (!aligned16(conv) || n_pos > 65535)
        return fail(QKK_EINVAL, "qkk_dn_step_seq: conv must be 16-byte aligned and n_pos at most 65535");
    hipLaunchKernelGGL(dn_step_seq_kernel, dim3(hV * (DN_DS / SEQ_RB)), dim3(128), 0, as_stream(stream), conv, gb, state, att,
                       hK, hV, kdiv, n_pos);
    hipLaunchKernelGGL(dn_gate_seq_kernel, dim3(hV, n_pos), dim3(DN_DS), 0, as_stream(stream), att, norm_w, z, hV, eps);
    return check_launch("qkk_dn_step_seq");
}

int qkk_dn_step(const float* conv, const float* gb, float* state, const float* norm_w, const float* z, float* att,
                uint32_t d_state, uint32_t hK, uint32_t hV, uint32_t kdiv, float eps, uint32_t n_slots, void* stream)
{
    if (!conv || !gb || !state || !norm_w || !z || !att) return fail(QKK_EINVAL, "qkk_dn_step: null pointer");
    if (int rc = check_slots("qkk_dn_step", n_slots)) return rc;
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "qkk_dn_step: state size %u not supported (128)", d_state);
    if (hK < 1 || hV < 1 || hV > 65535 || hK > 65535) return fail(QKK_ESHAPE, "qkk_dn_step: head counts out of range");
    if (kdiv ? (hV + kdiv - 1) / kdiv > hK : false)
        return fail(QKK_ESHAPE, "qkk_dn_step: %u value heads / %u exceed %u key heads", hV, kdiv, hK);
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_dn_step: eps must be non-negative");
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(dn_step_kernel, dim3(hV, n_slots), dim3(DN_DS * DN_PARTS), 0, as_stream(stream), conv, gb, state,
                       norm_w, z, att, hK, hV, kdiv, eps);
    return check_launch("qkk_dn_step");
}

int qkk_dn_step_fused(const float* x, const float* w_norm, float norm_eps, const float* alpha_w, const float* beta_w,
                      const float* dt_bias, const float* a_vec, uint32_t n_embd, float* conv_state, const float* qkv,
                      const float* ker, float* state, const float* norm_w, const float* z, float* att, uint32_t d_state,
                      uint32_t hK, uint32_t hV, uint32_t kdiv, float eps, uint32_t n_slots, void* stream)
{
    const char* who = "qkk_dn_step_fused";
    if (!x || !alpha_w || !beta_w || !dt_bias || !a_vec || !conv_state || !qkv || !ker || !state || !norm_w || !z || !att)
        return fail(QKK_EINVAL, "%s: null pointer", who);
    if (int rc = check_slots(who, n_slots)) return rc;
    if (n_embd != 2048) return fail(QKK_ESHAPE, "%s: n_embd %u not supported (2048)", who, n_embd);
    if (d_state != DN_DS) return fail(QKK_ESHAPE, "%s: state size %u not supported (128)", who, d_state);
    if (hK < 1 || hK > 32767 || hV != 2 * hK || (kdiv != 0 && kdiv != 2))
        return fail(QKK_ESHAPE, "%s: two value heads per key head are required (got %u on %u, kdiv %u)", who, hV, hK, kdiv);
    if (!aligned16(x) || !aligned16(alpha_w) || !aligned16(beta_w) || !aligned16(ker) || (w_norm && !aligned16(w_norm)))
        return fail(QKK_EINVAL, "%s: x, the weight rows, ker and w_norm must be 16-byte aligned", who);
    if (!(eps >= 0.f) || !(norm_eps >= 0.f)) return fail(QKK_EINVAL, "%s: eps must be non-negative", who);
    if (int rc = require_device()) return rc;
    const dim3 grid(hK, n_slots), block(DN_DS * DN_PARTS);
    if (w_norm)
        hipLaunchKernelGGL((dn_fused_step_kernel<8, true>), grid, block, 0, as_stream(stream), conv_state, qkv, ker, x, w_norm,
                           norm_eps, alpha_w, beta_w, dt_bias, a_vec, state, norm_w, z, att, hK, hV, kdiv, eps);
    else
        hipLaunchKernelGGL((dn_fused_step_kernel<8, false>), grid, block, 0, as_stream(stream), conv_state, qkv, ker, x,
                           (const float*)nullptr, 0.f, alpha_w, beta_w, dt_bias, a_vec, state, norm_w, z, att, hK, hV, kdiv,
                           eps);
    return check_launch(who);
}

} // extern "C"
