// qk_glue.hip -- the fp32 glue between the projections of a layer: residual adds fused with
// RMS norm, plain vector add, embedding-row lookup.
//   v = a [+ b [+ c]]            summed left to right in fp32, optionally stored (next residual)
//   xn = v * scale * w,  scale = 1 / sqrt(mean(v^2) + eps)
// (reference shaders/rmsnorm.comp:19-32, add_rmsnorm.comp:23-40, add_rms3.comp:24-41,
//  vec_add.comp:13-14; host src/main.cpp:4194, 4379-4402.)
// One workgroup of four waves per activation row, as in the reference; a row of up to 8192
// floats is read once and stays in registers between the sum of squares and the scaling.
// The outputs may be the inputs (in-place residual update or norm): every element is read
// and written by the same thread, reads first; only w must not overlap an output.
#include "qk_device.h"
#include "qk_host.h"

#include <algorithm>

namespace qk {

// Rows of n floats, n % 4 == 0, n <= 1024 * VPT, all pointers 16-byte aligned.
template <int NIN, int VPT>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(const float* a, const float* b, const float* c,
                                                          const float* __restrict__ w, float* sum_out, float* xn,
                                                          uint32_t n, float eps)
{
    __shared__ float s_red[4];
    const size_t base = (size_t)blockIdx.x * n;
    const uint32_t quads = n / 4;
    float4 v[VPT], g[VPT]; // the norm weights travel with the row: one round trip, not two
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; j++) {
        const uint32_t q = threadIdx.x + 256u * j;
        float4 t = float4{0.f, 0.f, 0.f, 0.f};
        g[j] = t;
        if (q < quads) {
            g[j] = *(const float4*)(w + 4 * (size_t)q);
            t = *(const float4*)(a + base + 4 * (size_t)q);
            if (NIN >= 2) {
                const float4 u = *(const float4*)(b + base + 4 * (size_t)q);
                t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
            }
            if (NIN >= 3) {
                const float4 u = *(const float4*)(c + base + 4 * (size_t)q);
                t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
            }
            if (sum_out) *(float4*)(sum_out + base + 4 * (size_t)q) = t;
        }
        v[j] = t;
        ss += t.x * t.x;
        ss += t.y * t.y;
        ss += t.z * t.z;
        ss += t.w * t.w;
    }
    const float tot = block_sum4(ss, s_red);
    const float scale = 1.f / sqrtf(tot / (float)n + eps);
#pragma unroll
    for (int j = 0; j < VPT; j++) {
        const uint32_t q = threadIdx.x + 256u * j;
        if (q < quads)
            *(float4*)(xn + base + 4 * (size_t)q) = float4{v[j].x * scale * g[j].x, v[j].y * scale * g[j].y,
                                                           v[j].z * scale * g[j].z, v[j].w * scale * g[j].w};
    }
}

// Any n, any alignment: two passes over the inputs, one float per access.
template <int NIN>
__global__ __launch_bounds__(256) void add_rmsnorm_any_kernel(const float* a, const float* b, const float* c,
                                                              const float* __restrict__ w, float* sum_out, float* xn,
                                                              uint32_t n, float eps)
{
    __shared__ float s_red[4];
    const size_t base = (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += 256u) {
        float t = a[base + i];
        if (NIN >= 2) t += b[base + i];
        if (NIN >= 3) t += c[base + i];
        if (sum_out) sum_out[base + i] = t;
        ss += t * t;
    }
    const float tot = block_sum4(ss, s_red);
    const float scale = 1.f / sqrtf(tot / (float)n + eps);
    for (uint32_t i = threadIdx.x; i < n; i += 256u) {
        float t;
        if (sum_out) t = sum_out[base + i]; // this thread stored it above
        else {
            t = a[base + i];
            if (NIN >= 2) t += b[base + i];
            if (NIN >= 3) t += c[base + i];
        }
        xn[base + i] = t * scale * w[i];
    }
}

__global__ __launch_bounds__(256) void vec_add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                      float* __restrict__ out, uint64_t n)
{
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256)
        out[i] = a[i] + b[i];
}

template <int NIN>
static void launch_norm(const float* a, const float* b, const float* c, const float* w, float* sum_out, float* xn,
                        uint32_t n, uint32_t rows, float eps, hipStream_t st)
{
    const bool vec = n % 4 == 0 && n <= 8192 && aligned16(a) && aligned16(w) && aligned16(xn) &&
                     (NIN < 2 || aligned16(b)) && (NIN < 3 || aligned16(c)) && (!sum_out || aligned16(sum_out));
    const dim3 grid(rows), block(256);
    if (!vec)
        hipLaunchKernelGGL(add_rmsnorm_any_kernel<NIN>, grid, block, 0, st, a, b, c, w, sum_out, xn, n, eps);
    else if (n <= 2048)
        hipLaunchKernelGGL((add_rmsnorm_kernel<NIN, 2>), grid, block, 0, st, a, b, c, w, sum_out, xn, n, eps);
    else if (n <= 4096)
        hipLaunchKernelGGL((add_rmsnorm_kernel<NIN, 4>), grid, block, 0, st, a, b, c, w, sum_out, xn, n, eps);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<NIN, 8>), grid, block, 0, st, a, b, c, w, sum_out, xn, n, eps);
}

// y = a + b, xn = y * scale(y) * w for `rows` rows (arguments already validated, launch not checked).
void launch_add_rmsnorm(const float* a, const float* b, const float* w, float* y, float* xn, uint32_t n, uint32_t rows,
                        float eps, hipStream_t st)
{
    launch_norm<2>(a, b, nullptr, w, y, xn, n, rows, eps, st);
}

static int norm_entry(const char* who, int nin, const float* a, const float* b, const float* c, const float* w,
                      float* sum_out, float* xn, uint32_t n, uint32_t rows, float eps, void* stream)
{
    if (!a || !w || !xn || (nin >= 2 && !b) || (nin >= 3 && !c)) return fail(QKK_EINVAL, "%s: null pointer", who);
    if (n == 0 || rows == 0) return fail(QKK_EINVAL, "%s: n and rows must be positive", who);
    if (rows > 65535u * 1024u) return fail(QKK_ESHAPE, "%s: %u rows is too many", who, rows);
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "%s: eps must be non-negative", who);
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    if (nin == 1) launch_norm<1>(a, nullptr, nullptr, w, sum_out, xn, n, rows, eps, st);
    else if (nin == 2) launch_norm<2>(a, b, nullptr, w, sum_out, xn, n, rows, eps, st);
    else launch_norm<3>(a, b, c, w, sum_out, xn, n, rows, eps, st);
    return check_launch(who);
}

} // namespace qk

using namespace qk;

extern "C" {

int qkk_rmsnorm(const float* x, const float* w, float* out, uint32_t n, uint32_t rows, float eps, void* stream)
{
    return norm_entry("qkk_rmsnorm", 1, x, nullptr, nullptr, w, nullptr, out, n, rows, eps, stream);
}

int qkk_add_rmsnorm(const float* a, const float* b, const float* w, float* y, float* xn, uint32_t n, uint32_t rows,
                    float eps, void* stream)
{
    if (!y) return fail(QKK_EINVAL, "qkk_add_rmsnorm: null pointer");
    return norm_entry("qkk_add_rmsnorm", 2, a, b, nullptr, w, y, xn, n, rows, eps, stream);
}

int qkk_add_rms3(const float* a, const float* b, const float* c, const float* w, float* s, float* xn, uint32_t n,
                 uint32_t rows, float eps, void* stream)
{
    if (!s) return fail(QKK_EINVAL, "qkk_add_rms3: null pointer");
    return norm_entry("qkk_add_rms3", 3, a, b, c, w, s, xn, n, rows, eps, stream);
}

int qkk_vec_add(const float* a, const float* b, float* out, uint64_t n, void* stream)
{
    if (!a || !b || !out) return fail(QKK_EINVAL, "qkk_vec_add: null pointer");
    if (n == 0) return QKK_OK;
    if (int rc = require_device()) return rc;
    const uint32_t grid = (uint32_t)std::min<uint64_t>((n + 255) / 256, persistent_blocks());
    hipLaunchKernelGGL(vec_add_kernel, dim3(grid), dim3(256), 0, as_stream(stream), a, b, out, n);
    return check_launch("qkk_vec_add");
}

} // extern "C"
