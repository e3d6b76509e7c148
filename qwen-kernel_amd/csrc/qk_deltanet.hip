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
// at 32 heads of 128).  Thread j owns row j, so both sums over i stay inside a thread; the state is
// kept COLUMN-major in memory -- element (row j, column i) at [i][j] -- so that the 64 lanes of a
// wave read 64 consecutive floats for every i (row-major, as in the reference, every lane would
// touch a cache line of its own per request).  A thread requests its whole row (dS loads) before
// any arithmetic: one memory round trip per head.
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

// grid (hV, slots), 128 threads: thread j = row j of the head's state.
__global__ __launch_bounds__(128) void dn_step_kernel(const float* __restrict__ conv, const float* __restrict__ gb,
                                                      float* __restrict__ state, const float* __restrict__ norm_w,
                                                      const float* __restrict__ z, float* __restrict__ att, uint32_t hK,
                                                      uint32_t hV, uint32_t kdiv, float eps)
{
    __shared__ float s_q[DN_DS], s_k[DN_DS];
    __shared__ float s_red[2];
    const uint32_t h = blockIdx.x, rq = blockIdx.y, j = threadIdx.x;
    const uint32_t kh = kdiv ? min(h / kdiv, hK - 1) : h % hK;
    const float* cv = conv + (size_t)rq * (2 * hK + hV) * DN_DS;
    float* S = state + ((size_t)rq * hV + h) * DN_DS * DN_DS; // column-major: (row j, column i) at [i][j]
    float s[DN_DS];
#pragma unroll
    for (uint32_t i = 0; i < DN_DS; i++) s[i] = S[(size_t)i * DN_DS + j];
    s_q[j] = cv[(size_t)kh * DN_DS + j] * (1.f / sqrtf((float)DN_DS));
    s_k[j] = cv[(size_t)(hK + kh) * DN_DS + j];
    const float vj = cv[(size_t)(2 * hK + h) * DN_DS + j];
    const float decay = expf(gb[(size_t)rq * 2 * hV + h]), beta = gb[(size_t)rq * 2 * hV + hV + h];
    const float zv = z[((size_t)rq * hV + h) * DN_DS + j], nw = norm_w[j];
    __syncthreads();
    float sk = 0.f;
#pragma unroll
    for (uint32_t i = 0; i < DN_DS; i++) sk += s[i] * s_k[i];
    const float dj = beta * (vj - sk * decay);
    float oj = 0.f;
#pragma unroll
    for (uint32_t i = 0; i < DN_DS; i++) {
        const float sn = s[i] * decay + s_k[i] * dj;
        S[(size_t)i * DN_DS + j] = sn;
        oj += sn * s_q[i];
    }
    const float scale = 1.f / sqrtf(block_sum2(oj * oj, s_red) / (float)DN_DS + eps);
    att[((size_t)rq * hV + h) * DN_DS + j] = oj * scale * nw * (zv / (1.f + expf(-zv)));
}

// The same two steps over n_pos consecutive positions of ONE slot in one launch each (reference
// shaders/dn_conv_batch.comp, dn_step_batch.comp + dn_gate_batch.comp): rows t of qkv / conv / gb /
// z / att are positions, the window and the state stay in registers from one position to the next
// and are written back once.  Per position the arithmetic is that of the one-position kernels; the
// next position's inputs are requested before the current one is worked on.  Shared arrays are
// double-buffered by the position's parity, so one barrier per use suffices.

// grid (channels / dS), 128 threads.
__global__ __launch_bounds__(128) void dn_conv_seq_kernel(float* __restrict__ st, const float* __restrict__ qkv,
                                                          const float* __restrict__ ker, float* __restrict__ out,
                                                          uint32_t channels, uint32_t qk_channels, float eps, uint32_t n_pos)
{
    __shared__ float s_red[2][2];
    const uint32_t ch = blockIdx.x * DN_DS + threadIdx.x;
    float* s = st + (size_t)ch * 3;
    float s0 = s[0], s1 = s[1], s2 = s[2];
    const float4 k = ((const float4*)ker)[ch];
    const bool unit = blockIdx.x * DN_DS < qk_channels; // a q or k head (uniform)
    float nxt = qkv[ch];
    for (uint32_t t = 0; t < n_pos; t++) {
        const float xin = nxt;
        if (t + 1 < n_pos) nxt = qkv[(size_t)(t + 1) * channels + ch];
        const float c = s0 * k.x + s1 * k.y + s2 * k.z + xin * k.w;
        float v = c / (1.f + expf(-c));
        s0 = s1; s1 = s2; s2 = xin;
        if (unit) v *= 1.f / fmaxf(sqrtf(block_sum2(v * v, s_red[t & 1u])), eps);
        out[(size_t)t * channels + ch] = v;
    }
    s[0] = s0; s[1] = s1; s[2] = s2;
}

// grid (hV), 128 threads: thread j = row j of the head's state, held in registers over all positions.
__global__ __launch_bounds__(128) void dn_step_seq_kernel(const float* __restrict__ conv, const float* __restrict__ gb,
                                                          float* __restrict__ state, const float* __restrict__ norm_w,
                                                          const float* __restrict__ z, float* __restrict__ att, uint32_t hK,
                                                          uint32_t hV, uint32_t kdiv, float eps, uint32_t n_pos)
{
    __shared__ float s_q[2][DN_DS], s_k[2][DN_DS];
    __shared__ float s_red[2][2];
    const uint32_t h = blockIdx.x, j = threadIdx.x;
    const uint32_t kh = kdiv ? min(h / kdiv, hK - 1) : h % hK;
    const size_t cstride = (size_t)(2 * hK + hV) * DN_DS;
    float* S = state + (size_t)h * DN_DS * DN_DS;
    float s[DN_DS];
#pragma unroll
    for (uint32_t i = 0; i < DN_DS; i++) s[i] = S[(size_t)i * DN_DS + j];
    const float nw = norm_w[j], q_scale = 1.f / sqrtf((float)DN_DS);
    float nq = conv[(size_t)kh * DN_DS + j], nk = conv[(size_t)(hK + kh) * DN_DS + j];
    float nv = conv[(size_t)(2 * hK + h) * DN_DS + j], ng = gb[h], nb = gb[hV + h], nz = z[(size_t)h * DN_DS + j];
    for (uint32_t t = 0; t < n_pos; t++) {
        const uint32_t b = t & 1u;
        s_q[b][j] = nq * q_scale;
        s_k[b][j] = nk;
        const float vj = nv, decay = expf(ng), beta = nb, zv = nz;
        if (t + 1 < n_pos) {
            const float* cv = conv + (size_t)(t + 1) * cstride;
            nq = cv[(size_t)kh * DN_DS + j];
            nk = cv[(size_t)(hK + kh) * DN_DS + j];
            nv = cv[(size_t)(2 * hK + h) * DN_DS + j];
            ng = gb[(size_t)(t + 1) * 2 * hV + h];
            nb = gb[(size_t)(t + 1) * 2 * hV + hV + h];
            nz = z[((size_t)(t + 1) * hV + h) * DN_DS + j];
        }
        __syncthreads();
        float sk = 0.f;
#pragma unroll
        for (uint32_t i = 0; i < DN_DS; i++) sk += s[i] * s_k[b][i];
        const float dj = beta * (vj - sk * decay);
        float oj = 0.f;
#pragma unroll
        for (uint32_t i = 0; i < DN_DS; i++) {
            const float sn = s[i] * decay + s_k[b][i] * dj;
            s[i] = sn;
            oj += sn * s_q[b][i];
        }
        const float scale = 1.f / sqrtf(block_sum2(oj * oj, s_red[b]) / (float)DN_DS + eps);
        att[((size_t)t * hV + h) * DN_DS + j] = oj * scale * nw * (zv / (1.f + expf(-zv)));
    }
#pragma unroll
    for (uint32_t i = 0; i < DN_DS; i++) S[(size_t)i * DN_DS + j] = s[i];
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
    hipLaunchKernelGGL(dn_conv_seq_kernel, dim3(channels / DN_DS), dim3(DN_DS), 0, as_stream(stream), conv_state, qkv, ker,
                       out, channels, qk_channels, eps, n_pos);
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
    hipLaunchKernelGGL(dn_step_seq_kernel, dim3(hV), dim3(DN_DS), 0, as_stream(stream), conv, gb, state, norm_w, z, att, hK,
                       hV, kdiv, eps, n_pos);
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
    hipLaunchKernelGGL(dn_step_kernel, dim3(hV, n_slots), dim3(DN_DS), 0, as_stream(stream), conv, gb, state, norm_w, z,
                       att, hK, hV, kdiv, eps);
    return check_launch("qkk_dn_step");
}

} // extern "C"
