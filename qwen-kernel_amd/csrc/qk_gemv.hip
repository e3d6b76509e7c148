// qk_gemv.hip -- block dequant-dot GEMVs for gfx950 and the bit-exact dequant kernel.
//
// y[b][m] = W[m] . x[b] on raw GGUF blocks.  One wave covers 2048 consecutive weights of a
// row per pass (one lane = 32 weights), keeps its slice of x in registers for every row it
// visits, fetches several rows before it starts the arithmetic so enough bytes are in
// flight, and reduces on DPP.  Rows shorter than 2048 share a wave (64/LPR rows per pass).
#include "qk_device.h"
#include "qk_host.h"

#include <stdarg.h>

#include <algorithm>

namespace qk {

// ---- host plumbing ---------------------------------------------------------------------

static thread_local char t_err[256] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_err, sizeof t_err, fmt, ap);
    va_end(ap);
    return code;
}

int require_device()
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(QKK_EDEVICE, "no HIP device: libqk.so has no CPU path");
    }
    return QKK_OK;
}

uint32_t persistent_blocks()
{
    static uint32_t cached = 0;
    if (cached == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached = (uint32_t)cus * 4u;
    }
    return cached;
}

int check_launch(const char* what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(QKK_EDEVICE, "%s: %s", what, hipGetErrorString(e));
    return QKK_OK;
}

// ---- bit-exact dequantisation ------------------------------------------------------------
// Software half -> float so NaN payloads and subnormals come out exactly as the CPU routine
// produces them (reference src/quants.h:12-34).
__device__ static float f16_bits_to_f32(uint32_t h)
{
    const uint32_t s = (h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u, m = h & 1023u, bits;
    if (e == 31u) bits = s | 0x7F800000u | (m << 13);
    else if (e != 0u) bits = s | ((e + 112u) << 23) | (m << 13);
    else if (m == 0u) bits = s;
    else {
        const int sh = __builtin_clz(m) - 21; // bring the leading one to bit 10
        m = (m << sh) & 1023u;
        bits = s | ((uint32_t)(113 - sh) << 23) | (m << 13);
    }
    return __builtin_bit_cast(float, bits);
}

__device__ static uint32_t rd16(const uint8_t* p) { return p[0] | ((uint32_t)p[1] << 8); }

// Value of element i (0 <= i < block size) of one block, products taken left to right as the
// CPU code writes them (reference src/quants.h:70-165).
template <int TYPE>
__device__ static float dequant_elem(const uint8_t* b, int i);

template <>
__device__ float dequant_elem<QKK_Q8_0>(const uint8_t* b, int i)
{
    return f16_bits_to_f32(rd16(b)) * (float)(int8_t)b[2 + i];
}
template <>
__device__ float dequant_elem<QKK_Q6_K>(const uint8_t* b, int i)
{
    const int n = i >> 7, c = (i >> 5) & 3, l = i & 31;
    const uint32_t lo = b[64 * n + 32 * (c & 1) + l];
    const int nib = c >= 2 ? (int)(lo >> 4) : (int)(lo & 15u);
    const int hi2 = (b[Q6_K_QH + 32 * n + l] >> (2 * c)) & 3;
    const int q = (nib | (hi2 << 4)) - 32;
    const float d = f16_bits_to_f32(rd16(b + Q6_K_D));
    const float sc = (float)(int8_t)b[Q6_K_SC + 8 * n + 2 * c + (l >> 4)];
    return d * sc * (float)q;
}
template <>
__device__ float dequant_elem<QKK_IQ4_XS>(const uint8_t* b, int i)
{
    constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
    const int ib = i >> 5, j = i & 15, hi = (i >> 4) & 1;
    const uint32_t sh = rd16(b + 2);
    const int ls = (int)(((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 15u) | (((sh >> (2 * ib)) & 3u) << 4));
    const float dl = f16_bits_to_f32(rd16(b)) * (float)(ls - 32);
    const uint32_t q = b[IQ4_XS_QS + 16 * ib + j];
    return dl * (float)kv[hi ? (q >> 4) : (q & 15u)];
}
template <>
__device__ float dequant_elem<QKK_IQ3_XXS>(const uint8_t* b, int i)
{
    const int ib = i >> 5, l = (i >> 3) & 3, half = (i >> 2) & 1, j = i & 3;
    const uint8_t* a = b + IQ3_XXS_AUX + 4 * ib;
    const uint32_t aux = a[0] | ((uint32_t)a[1] << 8) | ((uint32_t)a[2] << 16) | ((uint32_t)a[3] << 24);
    const float db = f16_bits_to_f32(rd16(b)) * (0.5f + (float)(aux >> 28)) * 0.5f;
    const uint32_t s7 = (aux >> (7 * l)) & 127u;
    const uint32_t sg = s7 | ((__builtin_popcount(s7) & 1u) << 7);
    const uint32_t cw = g_iq3xxs_grid[b[IQ3_XXS_QS + 8 * ib + 2 * l + half]];
    const float mag = (float)((cw >> (8 * j)) & 255u);
    return db * mag * (((sg >> (4 * half + j)) & 1u) ? -1.f : 1.f);
}

template <int TYPE, int BLOCK_ELEMS, int BLOCK_BYTES>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ W,
                                                      float* __restrict__ out, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint64_t blk = i / BLOCK_ELEMS;
    out[i] = dequant_elem<TYPE>(W + blk * BLOCK_BYTES, (int)(i % BLOCK_ELEMS));
}

// Embedding lookup: row ids[idx + per_req * rq] of the token-embedding tensor, dequantised with the
// same element routine (bit-exact), into activation row rq (reference shaders/embed_q6k.comp:27-49,
// embed_q8_0.comp:24-34).  A token id outside the vocabulary reads the last row instead of memory
// outside the tensor.
template <int TYPE, int BLOCK_ELEMS, int BLOCK_BYTES>
__global__ __launch_bounds__(256) void embed_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ ids,
                                                    uint32_t idx, uint32_t per_req, float* __restrict__ x,
                                                    uint32_t kdim, uint32_t n_vocab)
{
    const uint32_t rq = blockIdx.y;
    const uint32_t tok = min(ids[idx + per_req * rq], n_vocab - 1);
    const uint8_t* row = W + (size_t)tok * (kdim / BLOCK_ELEMS) * BLOCK_BYTES;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < kdim; i += gridDim.x * 256)
        x[(size_t)rq * kdim + i] = dequant_elem<TYPE>(row + (size_t)(i / BLOCK_ELEMS) * BLOCK_BYTES, (int)(i % BLOCK_ELEMS));
}

__global__ __launch_bounds__(256) void dequant_f16_kernel(const uint16_t* __restrict__ W,
                                                          float* __restrict__ out, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = f16_bits_to_f32(W[i]);
}

// ---- quantised GEMV ---------------------------------------------------------------------
// LPR   lanes per row (8..64): a row of K = 32*LPR*PASSES weights.
// PASSES how many 32*LPR slices a row has; x slices for all passes stay in registers.
// RIF   rows in flight per lane group: loads of RIF rows are issued before any arithmetic.
// DEEP  true: two register sets, the next chunk's loads in flight during the arithmetic of the
//       current one (large matrices); false: one chunk at a time (a wave has one or two chunks).
template <int TYPE, int LPR, int PASSES, int RIF, bool DEEP>
__global__ __launch_bounds__(256) void gemv_q_kernel(const uint8_t* __restrict__ W,
                                                     const float* __restrict__ X,
                                                     float* __restrict__ Y, uint32_t M, uint32_t K,
                                                     uint32_t row_bytes)
{
    __shared__ IqTables tab;
    constexpr bool TABLES = TYPE == QKK_IQ3_XXS || TYPE == QKK_IQ4_XS;
    // the codebook word travels with the first round trip (activations, first rows) and goes to LDS
    // after those loads are issued: a fill and a barrier up front would be a round trip of their own
    uint32_t grid_word = 0;
    if constexpr (TABLES) grid_word = g_iq3xxs_grid[threadIdx.x];
    constexpr int GROUPS = WAVE / LPR; // rows a wave works on side by side
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;

    XSlice xs[PASSES];
    float xsum[PASSES][4];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        load_xslice<TYPE>(xs[p], x + p * 32 * LPR, lir);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) s += xs[p].v[c * 8 + i];
            xsum[p][c] = s;
        }
    }
    const uint32_t pass_bytes = row_bytes / PASSES;

    // chunks of GROUPS*RIF rows are dealt round-robin to the waves of the (persistent) grid;
    // the loads of a wave's next chunk are issued before the arithmetic of the current one
    // (two register sets, loop unrolled by two, no branch around the loads: chunks past the
    // end re-read the last row and their results are dropped)
    constexpr uint32_t CHUNK = GROUPS * RIF;
    const uint32_t stride = gridDim.x * 4 * CHUNK;
    LaneW<TYPE> w[DEEP ? 2 : 1][RIF][PASSES];
    auto fetch = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            const uint32_t r = min(r0 + i * GROUPS + grp, M - 1);
#pragma unroll
            for (int p = 0; p < PASSES; p++)
                w[set][i][p].load(W + (size_t)r * row_bytes + (size_t)p * pass_bytes, lir);
        }
    };
    auto reduce = [&](int set, uint32_t r0) {
#pragma unroll
        for (int i = 0; i < RIF; i++) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < PASSES; p++) acc += w[set][i][p].dot(xs[p], xsum[p], &tab, lir);
            acc = lanes_sum<LPR>(acc);
            const uint32_t r = r0 + i * GROUPS + grp;
            if (lir == 0 && r < M) y[r] = acc;
        }
    };
    uint32_t r0 = (blockIdx.x * 4 + wave) * CHUNK;
    if constexpr (TABLES || DEEP) fetch(0, r0); // rows past the end re-read the last row
    if constexpr (TABLES) {
        tab.grid[threadIdx.x] = grid_word;
        if (threadIdx.x < 16) {
            constexpr int8_t kv[16] = {QK_IQ4NL_VALUES};
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) v = (int)threadIdx.x == i ? (float)kv[i] : v;
            tab.iq4[threadIdx.x] = v;
        }
        __syncthreads();
    }
    if constexpr (DEEP) {
        for (; r0 < M; r0 += 2 * stride) {
            fetch(1, r0 + stride);
            reduce(0, r0);
            fetch(0, r0 + 2 * stride);
            reduce(1, r0 + stride);
        }
    } else if constexpr (TABLES) { // the first chunk is already on its way
        while (r0 < M) {
            reduce(0, r0);
            r0 += stride;
            if (r0 < M) fetch(0, r0); // wave-uniform
        }
    } else {
        for (; r0 < M; r0 += stride) {
            fetch(0, r0);
            reduce(0, r0);
        }
    }
}

// Any K that is a block multiple: one wave per row, x re-read from cache each pass.
template <int TYPE>
__global__ __launch_bounds__(256) void gemv_q_generic_kernel(const uint8_t* __restrict__ W,
                                                             const float* __restrict__ X,
                                                             float* __restrict__ Y, uint32_t M,
                                                             uint32_t K, uint32_t row_bytes)
{
    __shared__ IqTables tab;
    if constexpr (TYPE == QKK_IQ3_XXS || TYPE == QKK_IQ4_XS) {
        fill_iq_tables(tab, g_iq3xxs_grid, threadIdx.x, 256);
        __syncthreads();
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;
    // lane tasks of 32 weights; for the 256-weight formats a task index maps to
    // (block = t/8, part = t%8) exactly as inside a full pass
    const uint32_t tasks = K / 32;
    for (uint32_t r = blockIdx.x * 4 + wave; r < M; r += gridDim.x * 4) {
        float acc = 0.f;
        for (uint32_t t0 = 0; t0 < tasks; t0 += 64) {
            const uint32_t t = t0 + lane;
            if (t < tasks) {
                // bytes per 64 tasks = 2048 weights
                const uint8_t* base = W + (size_t)r * row_bytes + (size_t)(t0 / 64) * (row_bytes * 2048ull / K);
                XSlice xs;
                load_xslice<TYPE>(xs, x + t0 * 32, lane);
                float xsum[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    float s = 0.f;
#pragma unroll
                    for (int i = 0; i < 8; i++) s += xs.v[c * 8 + i];
                    xsum[c] = s;
                }
                LaneW<TYPE> w;
                w.load(base, lane);
                acc += w.dot(xs, xsum, &tab, lane);
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) y[r] = acc;
    }
}

// ---- dense rows (F16 / F32) ---------------------------------------------------------------
// One wave per row; a lane takes 16-byte chunks at a stride of 64 chunks.
template <typename T> // T = _Float16 or float
__global__ __launch_bounds__(256) void gemv_dense_kernel(const T* __restrict__ W,
                                                         const float* __restrict__ X,
                                                         float* __restrict__ Y, uint32_t M, uint32_t K)
{
    constexpr int PER = 16 / sizeof(T); // elements per 16-byte chunk
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;
    const uint32_t chunks = K / PER;
    for (uint32_t r = blockIdx.x * 4 + wave; r < M; r += gridDim.x * 4) {
        const uint4* row = (const uint4*)(W + (size_t)r * K);
        float acc0 = 0.f, acc1 = 0.f;
        for (uint32_t c = lane; c < chunks; c += 64) {
            const uint4 raw = row[c];
            const float4* xp = (const float4*)(x + (size_t)c * PER);
            if constexpr (sizeof(T) == 2) {
                const float4 xa = xp[0], xb = xp[1];
                const _Float16* h = (const _Float16*)&raw;
                acc0 += (float)h[0] * xa.x + (float)h[1] * xa.y + (float)h[2] * xa.z + (float)h[3] * xa.w;
                acc1 += (float)h[4] * xb.x + (float)h[5] * xb.y + (float)h[6] * xb.z + (float)h[7] * xb.w;
            } else {
                const float4 xa = xp[0];
                const float* f = (const float*)&raw;
                acc0 += f[0] * xa.x + f[1] * xa.y;
                acc1 += f[2] * xa.z + f[3] * xa.w;
            }
        }
        const float s = wave_sum(acc0 + acc1);
        if (lane == 0) y[r] = s;
    }
}

// ---- launchers ----------------------------------------------------------------------------

template <int TYPE, int LPR, int PASSES, int RIF>
static void launch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch,
                     uint32_t row_bytes, hipStream_t st)
{
    constexpr uint32_t CHUNK = WAVE / LPR * RIF;
    const uint32_t waves = (M + CHUNK - 1) / CHUNK;
    const dim3 grid(std::min((waves + 3) / 4, persistent_blocks()), batch);
    if (waves > 4 * grid.x * 4) // at least four chunks per wave: worth the second register set
        hipLaunchKernelGGL((gemv_q_kernel<TYPE, LPR, PASSES, RIF, true>), grid, dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, row_bytes);
    else
        hipLaunchKernelGGL((gemv_q_kernel<TYPE, LPR, PASSES, RIF, false>), grid, dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, row_bytes);
}

template <int TYPE>
static int dispatch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch,
                      hipStream_t st)
{
    const uint32_t rb = (uint32_t)qkk_row_bytes(TYPE, K);
    constexpr uint32_t MINK = TYPE == QKK_Q8_0 ? 32 : 256;
    // rows per wave: four where the matrix has rows enough to give every CU several waves that way,
    // fewer for short matrices (512 rows: 3.1-3.4 us with one row per wave against 4.6-5.2 us with four)
    // a layer's input projections as one matrix (12288 = qkv + gate, 9216 = q + k + v rows): M / 1024 rows
    // per wave make 256 workgroups, one per CU, where eight leave half the CUs with a second one
    if (K == 2048 && M == 12288 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 12>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M == 9216 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 9>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M >= 8192 && TYPE == QKK_Q8_0) launch_q<TYPE, 64, 1, 8>(W, X, Y, M, K, batch, rb, st); // 7.5 -> 6.9 us
    else if (K == 2048 && M >= 2048) launch_q<TYPE, 64, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048 && M >= 1024) launch_q<TYPE, 64, 1, 2>(W, X, Y, M, K, batch, rb, st);
    else if (K == 2048) launch_q<TYPE, 64, 1, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 4096 && M >= 1024) launch_q<TYPE, 64, 2, 2>(W, X, Y, M, K, batch, rb, st);
    else if (K == 4096) launch_q<TYPE, 64, 2, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 8192) launch_q<TYPE, 64, 4, 1>(W, X, Y, M, K, batch, rb, st);
    else if (K == 1024) launch_q<TYPE, 32, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 512) launch_q<TYPE, 16, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else if (K == 256) launch_q<TYPE, 8, 1, 4>(W, X, Y, M, K, batch, rb, st);
    else {
        (void)MINK;
        const uint32_t blocks = (uint32_t)std::min<uint64_t>(((uint64_t)M + 3) / 4, 4096);
        hipLaunchKernelGGL((gemv_q_generic_kernel<TYPE>), dim3(blocks, batch), dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, rb);
    }
    return check_launch("qkk_gemv");
}

} // namespace qk

using namespace qk;

namespace qk {
bool coop_gemm_launch(int type, const uint8_t* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t N,
                      hipStream_t st);
// rows from which the weights are read once for all rows on the matrix cores; K = 4096 takes two
// passes there (13 us at 2048 x 4096 whatever the batch), so one more row stays on one pass per row
constexpr uint32_t COOP_MIN_BATCH = 3, COOP_MIN_BATCH_K4096 = 4;
void* moe_static_scratch();
} // namespace qk

extern "C" {

const char* qkk_last_error(void) { return t_err; }

int qkk_device_info(char* arch_host, size_t arch_len, uint32_t* n_cu_host)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    if (arch_host && arch_len) arch_host[0] = 0;
    if (n_cu_host) *n_cu_host = 0;
    if (n > 0) {
        hipDeviceProp_t p;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) {
            if (arch_host && arch_len) snprintf(arch_host, arch_len, "%s", p.gcnArchName);
            if (n_cu_host) *n_cu_host = (uint32_t)p.multiProcessorCount;
        }
        (void)moe_static_scratch(); // set-up for qkk_moe_decode_static on the current device
    }
    return n;
}

size_t qkk_row_bytes(int type, uint64_t k)
{
    switch (type) {
    case QKK_F32: return (size_t)k * 4;
    case QKK_F16: return (size_t)k * 2;
    case QKK_Q8_0: return k % 32 ? 0 : (size_t)(k / 32) * Q8_0_BYTES;
    case QKK_Q6_K: return k % 256 ? 0 : (size_t)(k / 256) * Q6_K_BYTES;
    case QKK_IQ4_XS: return k % 256 ? 0 : (size_t)(k / 256) * IQ4_XS_BYTES;
    case QKK_IQ3_XXS: return k % 256 ? 0 : (size_t)(k / 256) * IQ3_XXS_BYTES;
    default: return 0;
    }
}

int qkk_dequant(int type, const void* W, float* out, uint64_t n, void* stream)
{
    if (!W || !out) return fail(QKK_EINVAL, "qkk_dequant: null pointer");
    if (n == 0) return QKK_OK;
    const uint64_t be = type == QKK_Q8_0 ? 32 : (type == QKK_F16 || type == QKK_F32) ? 1 : 256;
    if (n % be) return fail(QKK_ESHAPE, "qkk_dequant: %llu elements is not a multiple of the block size %llu",
                            (unsigned long long)n, (unsigned long long)be);
    if (n > 0xFFFFFFFFull * 256ull) return fail(QKK_ESHAPE, "qkk_dequant: too many elements");
    if (int rc = require_device()) return rc;
    const dim3 grid((uint32_t)((n + 255) / 256));
    hipStream_t st = as_stream(stream);
    const uint8_t* w = (const uint8_t*)W;
    switch (type) {
    case QKK_Q8_0: hipLaunchKernelGGL((dequant_kernel<QKK_Q8_0, 32, Q8_0_BYTES>), grid, dim3(256), 0, st, w, out, n); break;
    case QKK_Q6_K: hipLaunchKernelGGL((dequant_kernel<QKK_Q6_K, 256, Q6_K_BYTES>), grid, dim3(256), 0, st, w, out, n); break;
    case QKK_IQ4_XS: hipLaunchKernelGGL((dequant_kernel<QKK_IQ4_XS, 256, IQ4_XS_BYTES>), grid, dim3(256), 0, st, w, out, n); break;
    case QKK_IQ3_XXS: hipLaunchKernelGGL((dequant_kernel<QKK_IQ3_XXS, 256, IQ3_XXS_BYTES>), grid, dim3(256), 0, st, w, out, n); break;
    case QKK_F16: hipLaunchKernelGGL(dequant_f16_kernel, grid, dim3(256), 0, st, (const uint16_t*)W, out, n); break;
    case QKK_F32:
        if (hipMemcpyAsync(out, W, n * 4, hipMemcpyDeviceToDevice, st) != hipSuccess)
            return check_launch("qkk_dequant(F32)");
        return QKK_OK;
    default: return fail(QKK_ETYPE, "qkk_dequant: unsupported tensor type %d", type);
    }
    return check_launch("qkk_dequant");
}

int qkk_embed(int type, const void* W, uint32_t n_vocab, uint32_t kdim, const uint32_t* ids, uint32_t n_ids,
              uint32_t idx, uint32_t per_req, float* x, uint32_t rows, void* stream)
{
    if (!W || !ids || !x) return fail(QKK_EINVAL, "qkk_embed: null pointer");
    if (n_vocab == 0 || kdim == 0 || rows == 0) return fail(QKK_EINVAL, "qkk_embed: n_vocab, kdim and rows must be positive");
    if (rows > 65535) return fail(QKK_ESHAPE, "qkk_embed: %u rows exceeds 65535", rows);
    if ((uint64_t)idx + (uint64_t)per_req * (rows - 1) >= n_ids)
        return fail(QKK_ESHAPE, "qkk_embed: ids[%u + %u*%u] is outside the %u ids", idx, per_req, rows - 1, n_ids);
    if (type != QKK_Q8_0 && type != QKK_Q6_K && type != QKK_IQ4_XS && type != QKK_IQ3_XXS)
        return fail(QKK_ETYPE, "qkk_embed: unsupported tensor type %d", type);
    if (qkk_row_bytes(type, kdim) == 0) return fail(QKK_ESHAPE, "qkk_embed: type %d with kdim=%u is not supported", type, kdim);
    if (int rc = require_device()) return rc;
    const dim3 grid(std::min((kdim + 255) / 256, 64u), rows);
    hipStream_t st = as_stream(stream);
    const uint8_t* w = (const uint8_t*)W;
    switch (type) {
    case QKK_Q8_0:
        hipLaunchKernelGGL((embed_kernel<QKK_Q8_0, 32, Q8_0_BYTES>), grid, dim3(256), 0, st, w, ids, idx, per_req, x, kdim, n_vocab);
        break;
    case QKK_Q6_K:
        hipLaunchKernelGGL((embed_kernel<QKK_Q6_K, 256, Q6_K_BYTES>), grid, dim3(256), 0, st, w, ids, idx, per_req, x, kdim, n_vocab);
        break;
    case QKK_IQ4_XS:
        hipLaunchKernelGGL((embed_kernel<QKK_IQ4_XS, 256, IQ4_XS_BYTES>), grid, dim3(256), 0, st, w, ids, idx, per_req, x, kdim, n_vocab);
        break;
    default:
        hipLaunchKernelGGL((embed_kernel<QKK_IQ3_XXS, 256, IQ3_XXS_BYTES>), grid, dim3(256), 0, st, w, ids, idx, per_req, x, kdim, n_vocab);
        break;
    }
    return check_launch("qkk_embed");
}

int qkk_gemv(int type, const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch,
             void* stream)
{
    if (!W || !X || !Y) return fail(QKK_EINVAL, "qkk_gemv: null pointer");
    if (M == 0 || K == 0 || batch == 0) return fail(QKK_EINVAL, "qkk_gemv: M, K and batch must be positive");
    if (batch > 65535) return fail(QKK_ESHAPE, "qkk_gemv: batch %u exceeds 65535", batch);
    if (!aligned16(W) || !aligned16(X)) return fail(QKK_EINVAL, "qkk_gemv: W and X must be 16-byte aligned");
    if (qkk_row_bytes(type, K) == 0)
        return fail(type == QKK_F32 || type == QKK_F16 || type == QKK_Q8_0 || type == QKK_Q6_K ||
                            type == QKK_IQ4_XS || type == QKK_IQ3_XXS
                        ? QKK_ESHAPE : QKK_ETYPE,
                    "qkk_gemv: type %d with K=%u is not supported", type, K);
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    // several rows: read the weights once for all of them on the matrix cores (needs Y aligned
    // like any output of that path); one row, or a shape that path does not cover: one pass per row
    if (batch >= (K >= 4096 ? COOP_MIN_BATCH_K4096 : COOP_MIN_BATCH) && aligned16(Y) && coop_gemm_launch(type, (const uint8_t*)W, X, Y, M, K, batch, st))
        return check_launch("qkk_gemv");
    switch (type) {
    case QKK_Q8_0: return dispatch_q<QKK_Q8_0>(W, X, Y, M, K, batch, st);
    case QKK_Q6_K: return dispatch_q<QKK_Q6_K>(W, X, Y, M, K, batch, st);
    case QKK_IQ4_XS: return dispatch_q<QKK_IQ4_XS>(W, X, Y, M, K, batch, st);
    case QKK_IQ3_XXS: return dispatch_q<QKK_IQ3_XXS>(W, X, Y, M, K, batch, st);
    case QKK_F16:
    case QKK_F32: {
        const uint32_t per = type == QKK_F16 ? 8 : 4;
        if (K % per) return fail(QKK_ESHAPE, "qkk_gemv: K=%u must be a multiple of %u for dense rows", K, per);
        const dim3 grid(std::min((M + 3) / 4, persistent_blocks()), batch);
        if (type == QKK_F16)
            hipLaunchKernelGGL(gemv_dense_kernel<_Float16>, grid, dim3(256), 0, st, (const _Float16*)W, X, Y, M, K);
        else
            hipLaunchKernelGGL(gemv_dense_kernel<float>, grid, dim3(256), 0, st, (const float*)W, X, Y, M, K);
        return check_launch("qkk_gemv");
    }
    default: return fail(QKK_ETYPE, "qkk_gemv: unsupported tensor type %d", type);
    }
}

} // extern "C"
