// qk_gemv.hip -- block dequant-dot GEMVs for gfx950 and the bit-exact dequant kernel.
//
// y[b][m] = W[m] . x[b] on raw GGUF blocks.  One wave covers 2048 consecutive weights of a
// row per pass (one lane = 32 weights), keeps its slice of x in registers for every row it
// visits, fetches several rows before it starts the arithmetic so enough bytes are in
// flight, and reduces on DPP.  Rows shorter than 2048 share a wave (64/LPR rows per pass).
#include "qk_device.h"
#include "qk_host.h"
#include "qk_stream.h"

#include <stdarg.h>

#include <stdlib.h>
#include <string.h>

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

namespace {
struct OptionDef {
    const char* name;
    const char* env;
    int Options::*field;
    int lo, hi;
};
const OptionDef OPTION_DEFS[] = {
    {"one_row", "QK_ONE_ROW", &Options::one_row_stream, 0, 1},   {"dense_reg", "QK_DENSE_REG", &Options::dense_reg, 0, 1},
    {"fused_norm", "QK_FUSED_NORM", &Options::fused_norm, 0, 1}, {"attn_block", "QK_ATTN_BLOCK", &Options::attn_block, 0, 1},
    {"dn_fused", "QK_DN_FUSED", &Options::dn_fused, 0, 1},       {"gemv_depth", "QK_GEMV_DEPTH", &Options::gemv_depth, 0, 16},
    {"head_depth", "QK_HEAD_DEPTH", &Options::head_depth, 0, 8}, {"rowwise_max", "QK_ROWWISE_MAX", &Options::rowwise_max, 0, 64},
    {"gemm_tiled", "QK_GEMM_TILED", &Options::gemm_tiled, 0, 1}, {"select_ranked", "QK_SELECT_RANKED", &Options::select_ranked, 0, 1},
    {"moe_rows", "QK_MOE_ROWS", &Options::moe_rows, 0, 1}, {"head_rows", "QK_HEAD_ROWS", &Options::head_rows, 0, 1},
};
} // namespace

// Applies the switches that are set in the environment right now (a value outside its range is ignored).
void apply_env_options(Options& v)
{
    for (const OptionDef& d : OPTION_DEFS) {
        const char* e = getenv(d.env);
        if (!e || !*e) continue;
        int x = atoi(e);
        if (d.field == &Options::one_row_stream) x = !strcmp(e, "stream") ? 1 : !strcmp(e, "lane") ? 0 : x;
        if (x >= d.lo && x <= d.hi) v.*d.field = x;
    }
}

Options& options()
{
    static Options o = [] {
        Options v;
        apply_env_options(v);
        return v;
    }();
    return o;
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
// K = 32 * LPR * PASSES.  LPR lanes (8..64) cover 32*LPR weights of a row, so 64/LPR rows lie side
// by side in a wave; PASSES (1, 2, 4) slices of 2048 weights make up longer rows (LPR = 64 then),
// the activation slices of all passes stay in registers.
// The rows are streamed (qk_stream.h): a wave takes chunks of RPC * 64/LPR consecutive rows -- one
// contiguous byte range, a multiple of 16 bytes for every format -- as 16-byte pieces through its own
// LDS area, the next chunk's loads in flight during the arithmetic of the current one.  A matrix of a
// few thousand chunks gets one chunk per wave, so that all of it is requested the moment the launch
// starts (a launch of this size is latency, not bandwidth); a larger one a persistent grid.  The rows
// behind the last full chunk are fetched per lane (the exact bytes: a partial chunk would end in a
// partial piece behind the tensor).  IQ3_XXS and IQ4_XS run their products on packed halves
// (LaneW::dot_h: LDS lookups that return signed half pairs, v_dot2_f32_f16 against the activations
// split into hi + lo halves); Q8_0 and Q6_K convert their integers (LaneW::dot).
template <int TYPE>
struct GemvShape {
    static constexpr bool HALF = TYPE == QKK_IQ3_XXS || TYPE == QKK_IQ4_XS;
    // rows of 2048 weights per chunk: about 3-4 KB in flight per wave
    static constexpr int RPC2048 = (TYPE == QKK_Q8_0 || TYPE == QKK_Q6_K) ? 2 : 4;
};

// NORM: the activation row is RMS-normalised on the way in, y = W . (x * nw / sqrt(mean(x^2) + eps)): the
// lanes that share a weight row hold all of x between them, so the mean square is one cross-lane sum and
// the dot products run on x * nw and are scaled at the end -- the norm costs no launch of its own.
template <int TYPE, int LPR, int PASSES, int RPC, bool NORM = false>
__global__ __launch_bounds__(256) void gemv_stream_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                          float* __restrict__ Y, uint32_t M,
                                                          const float* __restrict__ nw, float eps)
{
    constexpr int GROUPS = WAVE / LPR;
    constexpr uint32_t K = 32u * LPR * PASSES;
    constexpr uint32_t RB = (uint32_t)qkk_row_bytes_dev<TYPE>(K), PB = RB / PASSES;
    constexpr uint32_t CH = RPC * GROUPS, CB = CH * RB, NPC = CB / 16;
    constexpr int NP = (NPC + 63) / 64;
    constexpr bool HALF = GemvShape<TYPE>::HALF;
    static_assert(CB % 16 == 0, "a chunk of rows must be whole 16-byte pieces");
    static_assert(PASSES == 1 || LPR == 64, "several passes need whole waves per row");
    __shared__ __attribute__((aligned(16))) uint8_t s_stage[4][WaveStage<NP>::AREA + 16];
    __shared__ IqTables tab;        // Q8_0 / Q6_K take no table; the unused ones cost no LDS
    __shared__ Iq3HalfTables tab3;
    __shared__ Iq4PairTable tab4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lir = lane % LPR, grp = lane / LPR;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;
    const uint32_t n_full = M / CH, stride = gridDim.x * 4;
    uint32_t c = blockIdx.x * 4 + wave;

    // round trip 1: the first chunk, the activations, the codebook
    WaveStage<NP> st;
    if (c < n_full) st.fetch(W + (size_t)c * CB, NPC, lane);
    uint32_t grid_word = 0;
    if constexpr (TYPE == QKK_IQ3_XXS) grid_word = g_iq3xxs_grid[threadIdx.x];
    XSlice xs[HALF ? 1 : PASSES];
    XSliceH xh[HALF ? PASSES : 1];
    float xsum[PASSES][4];
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        XSlice f;
        load_xslice<TYPE>(f, x + p * 32 * LPR, lir);
        if constexpr (NORM) {
            XSlice g;
            load_xslice<TYPE>(g, nw + p * 32 * LPR, lir);
#pragma unroll
            for (int i = 0; i < 32; i++) {
                ss += f.v[i] * f.v[i];
                f.v[i] *= g.v[i];
            }
        }
        if constexpr (TYPE == QKK_IQ4_XS) split_xslice_iq4(xh[p], f);
        else if constexpr (HALF) split_xslice(xh[p], f);
        else {
            xs[p] = f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float t = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) t += f.v[q * 8 + i];
                xsum[p][q] = t;
            }
        }
    }
    if constexpr (TYPE == QKK_IQ3_XXS) fill_iq3_half_entry(tab3, threadIdx.x, grid_word);
    if constexpr (TYPE == QKK_IQ4_XS) fill_iq4_pair_entry(tab4, threadIdx.x);
    if constexpr (HALF) __syncthreads();
    float out_scale = 1.f;
    if constexpr (NORM) out_scale = 1.f / sqrtf(lanes_sum<LPR>(ss) / (float)K + eps);

    auto dot_row = [&](const LaneW<TYPE> (&w)[PASSES]) {
        float acc = 0.f;
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            if constexpr (TYPE == QKK_IQ3_XXS) acc += w[p].dot_h(xh[p], &tab3);
            else if constexpr (TYPE == QKK_IQ4_XS) acc += w[p].dot_h(xh[p], &tab4, lir);
            else acc += w[p].dot(xs[p], xsum[p], &tab, lir);
        }
        return lanes_sum<LPR>(acc) * out_scale;
    };

    uint8_t* area = s_stage[wave];
    vmem_drain(); // the activations have arrived: no wait for them inside the loop, behind the next chunk's loads
    for (; c < n_full; c += stride) {
        st.commit(area, lane);
        const uint32_t cn = c + stride;
        if (cn < n_full) st.fetch(W + (size_t)cn * CB, NPC, lane);
#pragma unroll
        for (int r = 0; r < RPC; r++) {
            const uint32_t in_chunk = r * GROUPS + grp;
            LaneW<TYPE> w[PASSES];
#pragma unroll
            for (int p = 0; p < PASSES; p++) lane_load_lds<TYPE>(w[p], area, in_chunk * RB + p * PB, lir);
            const float acc = dot_row(w);
            if (lir == 0) y[c * CH + in_chunk] = acc;
        }
    }
    // the rows behind the last full chunk, 64/LPR at a time, each lane fetching its own fields
    const uint32_t tail0 = n_full * CH, tail_groups = (M - tail0 + GROUPS - 1) / GROUPS;
    for (uint32_t t = blockIdx.x * 4 + wave; t < tail_groups; t += stride) {
        const uint32_t row = tail0 + t * GROUPS + grp;
        const uint8_t* rp = W + (size_t)min(row, M - 1) * RB; // lanes past the end re-read the last row
        LaneW<TYPE> w[PASSES];
#pragma unroll
        for (int p = 0; p < PASSES; p++) w[p].load(rp + (size_t)p * PB, lir);
        const float acc = dot_row(w);
        if (lir == 0 && row < M) y[row] = acc;
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

// The same rows for K = CPL * 64 chunks of 16 bytes exactly (K = 512 * CPL halves or 256 * CPL floats): the
// lane's share of x -- the chunks lane, lane + 64, ... -- stays in registers for every row the wave visits
// (re-read per row, x made up two thirds of the bytes through the L1: 8 KB of x for a 4 KB row of halves),
// and the next row's chunks are requested before the current row's arithmetic.  Same assignment of chunks
// to lanes and the same two partial sums as gemv_dense_kernel: the same bits.
template <typename T, int CPL>
__global__ __launch_bounds__(256) void gemv_dense_reg_kernel(const T* __restrict__ W, const float* __restrict__ X,
                                                             float* __restrict__ Y, uint32_t M)
{
    constexpr int PER = 16 / sizeof(T);
    constexpr uint32_t K = CPL * 64 * PER;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* x = X + (size_t)blockIdx.y * K;
    float* y = Y + (size_t)blockIdx.y * M;
    const uint32_t stride = gridDim.x * 4;
    uint32_t r = blockIdx.x * 4 + wave;
    if (r >= M) return; // the whole wave
    uint4 cur[CPL], nxt[CPL];
#pragma unroll
    for (int i = 0; i < CPL; i++) cur[i] = ((const uint4*)(W + (size_t)r * K))[lane + 64 * i];
    float xs[CPL][PER];
#pragma unroll
    for (int i = 0; i < CPL; i++) {
        const float4* xp = (const float4*)(x + (size_t)(lane + 64 * i) * PER);
#pragma unroll
        for (int q = 0; q < PER / 4; q++) {
            const float4 v = xp[q];
            xs[i][4 * q] = v.x; xs[i][4 * q + 1] = v.y; xs[i][4 * q + 2] = v.z; xs[i][4 * q + 3] = v.w;
        }
    }
    for (; r < M; r += stride) {
        const uint32_t rn = min(r + stride, M - 1); // past the end: a harmless re-read of the last row
#pragma unroll
        for (int i = 0; i < CPL; i++) nxt[i] = ((const uint4*)(W + (size_t)rn * K))[lane + 64 * i];
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < CPL; i++) {
            if constexpr (sizeof(T) == 2) {
                const _Float16* h = (const _Float16*)&cur[i];
                acc0 += (float)h[0] * xs[i][0] + (float)h[1] * xs[i][1] + (float)h[2] * xs[i][2] + (float)h[3] * xs[i][3];
                acc1 += (float)h[4] * xs[i][4] + (float)h[5] * xs[i][5] + (float)h[6] * xs[i][6] + (float)h[7] * xs[i][7];
            } else {
                const float* f = (const float*)&cur[i];
                acc0 += f[0] * xs[i][0] + f[1] * xs[i][1];
                acc1 += f[2] * xs[i][2] + f[3] * xs[i][3];
            }
        }
        const float sum = wave_sum(acc0 + acc1);
        if (lane == 0) y[r] = sum;
#pragma unroll
        for (int i = 0; i < CPL; i++) cur[i] = nxt[i];
    }
}

template <typename T>
static bool launch_dense_reg(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch, hipStream_t st)
{
    constexpr uint32_t PER = 16 / sizeof(T);
    if (K % (64 * PER)) return false;
    // four workgroups per CU and at least two rows per wave where there are that many: x is fetched once per
    // wave, so a wave that visits one row only has gained nothing over the chunk loop
    const dim3 grid(std::max(1u, std::min((M + 7) / 8, persistent_blocks())), batch);
    switch (K / (64 * PER)) {
    case 1: hipLaunchKernelGGL((gemv_dense_reg_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)W, X, Y, M); return true;
    case 2: hipLaunchKernelGGL((gemv_dense_reg_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)W, X, Y, M); return true;
    case 4: hipLaunchKernelGGL((gemv_dense_reg_kernel<T, 4>), grid, dim3(256), 0, st, (const T*)W, X, Y, M); return true;
    case 8: hipLaunchKernelGGL((gemv_dense_reg_kernel<T, 8>), grid, dim3(256), 0, st, (const T*)W, X, Y, M); return true;
    default: return false;
    }
}

// ---- launchers ----------------------------------------------------------------------------

template <int TYPE, int LPR, int PASSES, bool NORM = false>
static void launch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t batch, hipStream_t st,
                     const float* nw = nullptr, float eps = 0.f)
{
    constexpr int RPC = GemvShape<TYPE>::RPC2048 / PASSES > 0 ? GemvShape<TYPE>::RPC2048 / PASSES : 1;
    constexpr uint32_t CH = RPC * (WAVE / LPR);
    constexpr uint32_t RB = (uint32_t)qkk_row_bytes_dev<TYPE>(32u * LPR * PASSES);
    constexpr uint32_t NP = (CH * RB / 16 + 63) / 64;
    // workgroups a CU holds (LDS: the four waves' areas + tables; 160 KB per CU) and the depth of the persistent grid
    constexpr uint32_t WG_LDS = 4 * (NP * 1024 + 16) + 4096, RESIDENT = std::min<uint32_t>(8, 160 * 1024 / WG_LDS);
    constexpr uint32_t DEPTH = TYPE == QKK_Q8_0 ? std::min<uint32_t>(4, RESIDENT) : RESIDENT;
    const uint32_t cus = persistent_blocks() / 4;
    const uint32_t chunks = M / CH, tail_groups = (M - chunks * CH + WAVE / LPR - 1) / (WAVE / LPR);
    const uint32_t want = (std::max(chunks, tail_groups) + 3) / 4; // one chunk per wave
    // the "gemv_depth" switch: workgroups per CU of the persistent grid, for sweeps on the device
    const uint32_t depth_opt = (uint32_t)options().gemv_depth;
    const uint32_t depth = depth_opt ? std::min(depth_opt, RESIDENT) : DEPTH;
    const uint32_t blocks = std::max(1u, want <= cus * RESIDENT ? want : cus * depth);
    hipLaunchKernelGGL((gemv_stream_kernel<TYPE, LPR, PASSES, RPC, NORM>), dim3(blocks, batch), dim3(256), 0, st,
                       (const uint8_t*)W, X, Y, M, nw, eps);
}

bool lane_gemv_launch(int type, const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch, hipStream_t st); // qk_gemv_lane.hip

// The streaming form of one quantised GEMV launch; false for a K outside the tiled shapes.
template <int TYPE>
static bool stream_gemv_launch(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch, hipStream_t st)
{
    if (K == 2048) launch_q<TYPE, 64, 1>(W, X, Y, M, batch, st);
    else if (K == 4096) launch_q<TYPE, 64, 2>(W, X, Y, M, batch, st);
    else if (K == 8192) launch_q<TYPE, 64, 4>(W, X, Y, M, batch, st);
    else if (K == 1024) launch_q<TYPE, 32, 1>(W, X, Y, M, batch, st);
    else if (K == 512) launch_q<TYPE, 16, 1>(W, X, Y, M, batch, st);
    else if (K == 256) launch_q<TYPE, 8, 1>(W, X, Y, M, batch, st);
    else return false;
    return true;
}

template <int TYPE>
static int dispatch_q(const void* W, const float* X, float* Y, uint32_t M, uint32_t K, uint32_t batch,
                      hipStream_t st)
{
    const bool tiled = options().one_row_stream ? stream_gemv_launch<TYPE>(W, X, Y, M, K, batch, st)
                                                : lane_gemv_launch(TYPE, W, X, Y, M, K, batch, st);
    if (!tiled) { // any other K that is a block multiple
        const uint32_t blocks = (uint32_t)std::min<uint64_t>(((uint64_t)M + 3) / 4, 4096);
        hipLaunchKernelGGL((gemv_q_generic_kernel<TYPE>), dim3(blocks, batch), dim3(256), 0, st,
                           (const uint8_t*)W, X, Y, M, K, (uint32_t)qkk_row_bytes(TYPE, K));
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

int qkk_set_option(const char* name, int value)
{
    if (!name) return fail(QKK_EINVAL, "qkk_set_option: null name");
    for (const OptionDef& d : OPTION_DEFS)
        if (!strcmp(name, d.name)) {
            if (value < d.lo || value > d.hi)
                return fail(QKK_EINVAL, "qkk_set_option: %s = %d outside %d..%d", name, value, d.lo, d.hi);
            options().*d.field = value;
            return QKK_OK;
        }
    return fail(QKK_EINVAL, "qkk_set_option: no switch named '%s'", name);
}

int qkk_get_option(const char* name, int* value)
{
    if (!name || !value) return fail(QKK_EINVAL, "qkk_get_option: null pointer");
    for (const OptionDef& d : OPTION_DEFS)
        if (!strcmp(name, d.name)) {
            *value = options().*d.field;
            return QKK_OK;
        }
    return fail(QKK_EINVAL, "qkk_get_option: no switch named '%s'", name);
}

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
        if (!options().dense_reg) {} // the chunk loop below
        else if (type == QKK_F16 ? launch_dense_reg<_Float16>(W, X, Y, M, K, batch, st) : launch_dense_reg<float>(W, X, Y, M, K, batch, st))
            return check_launch("qkk_gemv");
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

int qkk_gemv_norm(int type, const void* W, const float* X, const float* w_norm, float eps, float* Y, uint32_t M,
                  uint32_t K, uint32_t batch, void* stream)
{
    if (!W || !X || !Y || !w_norm) return fail(QKK_EINVAL, "qkk_gemv_norm: null pointer");
    if (M == 0 || batch == 0) return fail(QKK_EINVAL, "qkk_gemv_norm: M and batch must be positive");
    if (batch > 16) return fail(QKK_ESHAPE, "qkk_gemv_norm: batch %u exceeds 16 (one pass over the weights per row)", batch);
    if (K != 2048) return fail(QKK_ESHAPE, "qkk_gemv_norm: K=%u not supported (2048)", K);
    if (!aligned16(W) || !aligned16(X) || !aligned16(w_norm))
        return fail(QKK_EINVAL, "qkk_gemv_norm: W, X and w_norm must be 16-byte aligned");
    if (!(eps >= 0.f)) return fail(QKK_EINVAL, "qkk_gemv_norm: eps must be non-negative");
    if (int rc = require_device()) return rc;
    hipStream_t st = as_stream(stream);
    switch (type) {
    case QKK_Q8_0: launch_q<QKK_Q8_0, 64, 1, true>(W, X, Y, M, batch, st, w_norm, eps); break;
    case QKK_Q6_K: launch_q<QKK_Q6_K, 64, 1, true>(W, X, Y, M, batch, st, w_norm, eps); break;
    case QKK_IQ4_XS: launch_q<QKK_IQ4_XS, 64, 1, true>(W, X, Y, M, batch, st, w_norm, eps); break;
    case QKK_IQ3_XXS: launch_q<QKK_IQ3_XXS, 64, 1, true>(W, X, Y, M, batch, st, w_norm, eps); break;
    default: return fail(QKK_ETYPE, "qkk_gemv_norm: tensor type %d is not a quantised block format", type);
    }
    return check_launch("qkk_gemv_norm");
}

} // extern "C"
