// qk_moe_grouped.hip -- routing for several tokens (decode slots or a prefill chunk): router
// logits, top-k selection and the grouping of (token, pick) pairs by expert.
//
// Each expert picked by at least one token is then visited once by the MFMA kernels of
// qk_moe_mfma.hip: its gate/up rows and its down rows cross HBM once however many tokens
// share it (the expert-major order of reference shaders/moe_gateup_iq3_grouped.comp:30-114 and
// moe_down_iq4_grouped.comp:24-75, driven by the pair lists of moe_group_pairs.comp).
// Launches of a step: route (router logits and -- in the workgroup that finishes last --
// selection + grouping; above 32 tokens a launch of its own that selects one token per wave
// and groups in its last workgroup), gate/up, down, fold.
#include "qk_moe_common.h"

#include <map>
#include <mutex>
#include <utility>
#include <algorithm>

namespace qk {

constexpr uint32_t SELECT_INLINE_MAX = 32; // up to this many tokens the route launch also selects

// The caller clears a workspace once; the arrival counter (word 0 of its 256-byte header) then returns to
// zero after every step, and no kernel ever writes the 63 words behind it.  Anything but zero there means
// the header was never cleared (or the clear, issued on another stream, has not completed): the counter
// cannot be trusted either, no workgroup may find itself last, and the step's numbers are wrong.  The
// routing launches look at those words and raise this flag (per device, sticky until
// qkk_moe_workspace_status reads it) so that the mistake is an error and not only wrong numbers.
static __device__ uint32_t g_ws_alarm;
__device__ __forceinline__ void check_ws_header(const MoeWs& ws, int lane)
{
    const uint32_t v = lane < 63 ? ws.counter[1 + lane] : 0u;
    if (__builtin_amdgcn_ballot_w64(v != 0u) != 0 && lane == 0) g_ws_alarm = 1u;
}

// ---- selection: one wave takes the tokens first, first+stride, ... TPW (1 or 2) at a time ---------
// (logits written by other workgroups: the caller's acquire fence, or a kernel boundary, precedes)
// my_log: TPW areas of LOG_AREA floats of LDS for this wave.  ids_lds: when not null the picks of
// token t are also left at ids_lds[16*t ..] for a grouping pass by the same workgroup.
constexpr uint32_t LOG_AREA = QKK_MAX_EXPERTS + 8;
template <int TPW>
__device__ static void select_tokens(const MoeWs& ws, qkk_sel* __restrict__ sel, MoeDims d, uint32_t N,
                                     uint32_t first, uint32_t stride, float* my_log, uint32_t* ids_lds, bool publish_ids)
{
    const int lane = threadIdx.x & 63;
    constexpr int NL = QKK_MAX_EXPERTS / 64 + 1;
    for (uint32_t t0 = first; t0 < N; t0 += TPW * stride) {
        // plain loads of the logits of all TPW tokens, issued before the first use: one round trip
        float lg[TPW][NL];
#pragma unroll
        for (int h = 0; h < TPW; h++) {
            const float* g = ws.logits + (size_t)min(t0 + h * stride, N - 1) * lstride(d.E);
#pragma unroll
            for (int i = 0; i < NL; i++) lg[h][i] = (uint32_t)(lane + 64 * i) <= d.E ? g[lane + 64 * i] : 0.f;
        }
#pragma unroll
        for (int h = 0; h < TPW; h++)
#pragma unroll
            for (int i = 0; i < NL; i++)
                if ((uint32_t)(lane + 64 * i) <= d.E) my_log[h * LOG_AREA + lane + 64 * i] = lg[h][i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int h = 0; h < TPW; h++) {
            const uint32_t t = t0 + h * stride;
            if (t >= N) break; // the whole wave
            const float* l = my_log + h * LOG_AREA;
            select_wave(l, d.E, d.k, &sel[t], ids_lds ? ids_lds + 16 * t : nullptr);
            if (lane == 0) sel[t].w_shared = 1.f / (1.f + expf(-l[d.E]));
            // a grouping workgroup elsewhere in the launch reads the ids: write them through
            if (publish_ids && (uint32_t)lane < d.k) publish(&sel[t].ids[lane], sel[t].ids[lane]);
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (publish_ids) publish_wait(); // acknowledged before the caller's barrier and arrival count
}

// ---- grouping of the N*k (token, pick) pairs by expert, by one workgroup of NW waves ----------
// ids: the picks of token t at ids_lds[16*t ..] when this workgroup selected them itself (LDS), else
// read from sel with loads that bypass the L1 (other workgroups of the launch published them).
// One expert per thread: counts by LDS atomics, exclusive offsets by a wave scan plus the sum of
// the earlier waves' totals, then the pairs are scattered behind per-expert LDS cursors.
template <int NW>
__device__ static void group_pairs_wg(const MoeWs& ws, qkk_sel* __restrict__ sel, const uint32_t* ids_lds, MoeDims d,
                                      uint32_t N, uint32_t* s_cnt, uint32_t* s_cur)
{
    static_assert(NW * 64 >= (int)QKK_MAX_EXPERTS, "one expert per thread");
    __shared__ uint32_t s_part[NW];
    const uint32_t e = threadIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    for (uint32_t i = threadIdx.x; i <= QKK_MAX_EXPERTS; i += NW * 64) s_cnt[i] = 0;
    __syncthreads();
    const uint32_t np = N * d.k;
    const volatile qkk_sel* vs = sel;
    const auto id_of = [&](uint32_t p) -> uint32_t {
        const uint32_t t = p / d.k, s = p % d.k;
        return min(ids_lds ? ids_lds[16 * t + s] : vs[t].ids[s], d.E - 1);
    };
    for (uint32_t p = threadIdx.x; p < np; p += NW * 64) atomicAdd(&s_cnt[id_of(p)], 1u);
    __syncthreads();
    // (pair count, "has pairs" flag) packed as count | flag << 20 (count <= 4096*16 < 2^20)
    const uint32_t c = e < d.E ? s_cnt[e] : 0u;
    const uint32_t mine = c | (c ? 1u << 20 : 0u);
    uint32_t incl = wave_incl_scan_u32(mine);
    if (lane == 63) s_part[wave] = incl;
    __syncthreads();
    for (uint32_t w = 0; w < wave; w++) incl += s_part[w];
    const uint32_t excl = incl - mine;
    const uint32_t off = excl & 0xFFFFFu, rank = excl >> 20;
    if (e < QKK_MAX_EXPERTS) s_cur[e] = off;
    if (e < d.E) {
        ws.offsets[e] = off;
        if (c) {
            ActiveExpert a{e, off, c, 0};
            ws.active[rank] = a;
        }
        if (e == d.E - 1) {
            ws.offsets[d.E] = off + c;
            *ws.n_active = rank + (c ? 1u : 0u);
        }
    }
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < np; p += NW * 64) {
        const uint32_t t = p / d.k, s = p % d.k;
        ws.pairs[min(atomicAdd(&s_cur[id_of(p)], 1u), np - 1)] = (t << 4) | s; // in range even if sel changes under us
    }
}

// ---- launch 1: router logits for N tokens ----------------------------------------------------
// One wave per task = (router row, group of TG tokens); row E is the shared-gate row.  All loads
// of a task -- the row and the TG activation rows -- are issued together: one memory round trip
// per task.  The router matrix is re-read once per token group (from L2 after the first).
template <int NCH>
__global__ __launch_bounds__(512) void moe_route_multi_kernel(const float* __restrict__ gate_inp,
                                                              const float* __restrict__ gate_inp_shexp,
                                                              const float* __restrict__ X, MoeWs ws,
                                                              qkk_sel* __restrict__ sel, MoeDims d, uint32_t N,
                                                              uint32_t select_here)
{
    constexpr int TG = NCH <= 8 ? 4 : 2; // tokens per task
    constexpr int NW = 8;                // waves per block
    __shared__ uint32_t s_last;
    __shared__ float s_log[NW * 2 * LOG_AREA];
    __shared__ uint32_t s_cnt[QKK_MAX_EXPERTS + 1], s_cur[QKK_MAX_EXPERTS + 1];
    __shared__ uint32_t s_ids[SELECT_INLINE_MAX * 16]; // the picks of every token, for the grouping below
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_rows = d.E + 1;
    const uint32_t task = blockIdx.x * NW + wave;
    const uint32_t t = task % n_rows, t0 = (task / n_rows) * TG;
    const uint32_t LS = lstride(d.E);
    if (select_here && blockIdx.x == 0 && wave == 0) check_ws_header(ws, lane);

    if (t0 < N) {
        const float4* row = (const float4*)(t < d.E ? gate_inp + (size_t)t * d.H : gate_inp_shexp);
        float4 w[NCH], xx[TG][NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
#pragma unroll
        for (int j = 0; j < TG; j++) {
            const float4* xv = (const float4*)(X + (size_t)min(t0 + j, N - 1) * d.H);
#pragma unroll
            for (int i = 0; i < NCH; i++) xx[j][i] = xv[lane + 64 * i];
        }
#pragma unroll
        for (int j = 0; j < TG; j++) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                a0 += w[i].x * xx[j][i].x + w[i].y * xx[j][i].y;
                a1 += w[i].z * xx[j][i].z + w[i].w * xx[j][i].w;
            }
            const float s = wave_sum(a0 + a1);
            if (lane == 0 && t0 + j < N) publish(&ws.logits[(size_t)(t0 + j) * LS + t], s);
        }
    }
    if (!select_here) return;

    publish_wait(); // every wave's logits are acknowledged before the arrival is counted
    __syncthreads();
    if (threadIdx.x == 0) s_last = arrive_last(&ws.counter[0], gridDim.x) ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        select_tokens<2>(ws, sel, d, N, wave, NW, s_log + (size_t)wave * 2 * LOG_AREA, s_ids, false);
        group_pairs_wg<NW>(ws, sel, s_ids, d, N, s_cnt, s_cur);
        if (threadIdx.x == 0) ws.counter[0] = 0u;
    }
}

// ---- router logits for many tokens --------------------------------------------------------------
// Workgroup = 8 router rows x 16 tokens: the 16 activation rows are staged in LDS once and every
// wave holds one router row in registers, so a row and an activation row cross the L1 once per
// workgroup instead of once per dot product.  Same arithmetic, in the same order, as
// moe_route_multi_kernel: a token's logits do not depend on how many tokens ride along.
constexpr uint32_t LOGITS_TILE_TOKENS = 16;
// Grid = (groups of 8 router rows) x (token tiles).  At 256 experts the shared-gate row (row E) makes
// a 33rd, nearly empty row group; where that pushes the grid past one workgroup per CU (128 tokens:
// 264 workgroups, a second round for eight of them) the launcher sets `ride`, and the row rides
// along instead: in every token tile one workgroup's wave 0 takes it as a second row.
template <bool RIDE>
__global__ __launch_bounds__(512) void moe_logits_tiled_kernel(const float* __restrict__ gate_inp,
                                                               const float* __restrict__ gate_inp_shexp,
                                                               const float* __restrict__ X, MoeWs ws, MoeDims d,
                                                               uint32_t N)
{
    QK_DYN_LDS(float, s_x); // [16][2048]
    constexpr int NCH = 8;                                      // n_embd = 2048: eight float4 per lane
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_rows = RIDE ? d.E : d.E + 1; // rows dealt out in groups of eight
    const uint32_t rgroups = (n_rows + 7) / 8;
    const uint32_t rg = blockIdx.x % rgroups, tt = blockIdx.x / rgroups;
    const uint32_t r = rg * 8 + wave, t0 = tt * LOGITS_TILE_TOKENS;
    const uint32_t nt = min(LOGITS_TILE_TOKENS, N - t0);
    const uint32_t LS = lstride(d.E);
    const bool extra = RIDE && wave == 0 && rg == tt % rgroups; // this wave also takes the shared-gate row
    if (blockIdx.x == 0 && wave == 0) check_ws_header(ws, lane); // the selection launch behind this one counts arrivals

    const float4* xs = (const float4*)(X + (size_t)t0 * 2048); // nt consecutive rows: one contiguous range
    float4 xv[LOGITS_TILE_TOKENS];
#pragma unroll
    for (uint32_t i = 0; i < LOGITS_TILE_TOKENS; i++) xv[i] = xs[min(threadIdx.x + 512 * i, nt * 512 - 1)];
    float4 w[NCH], w2[NCH];
    const float4* row = (const float4*)(r < d.E ? gate_inp + (size_t)r * 2048 : gate_inp_shexp); // row E = shared gate
    const float4* row2 = (const float4*)gate_inp_shexp;
#pragma unroll
    for (int i = 0; i < NCH; i++) w[i] = row[lane + 64 * i];
    if constexpr (RIDE) {
#pragma unroll
        for (int i = 0; i < NCH; i++) w2[i] = extra ? row2[lane + 64 * i] : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (uint32_t i = 0; i < LOGITS_TILE_TOKENS; i++) ((float4*)s_x)[threadIdx.x + 512 * i] = xv[i];
    __syncthreads();
    if (r >= n_rows) return;
    for (uint32_t t = 0; t < nt; t++) {
        float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const float4 x = ((const float4*)s_x)[t * 512 + lane + 64 * i];
            a0 += w[i].x * x.x + w[i].y * x.y;
            a1 += w[i].z * x.z + w[i].w * x.w;
            if constexpr (RIDE) {
                if (extra) { // wave-uniform
                    b0 += w2[i].x * x.x + w2[i].y * x.y;
                    b1 += w2[i].z * x.z + w2[i].w * x.w;
                }
            }
        }
        const float sum = wave_sum(a0 + a1);
        if (lane == 0) ws.logits[(size_t)(t0 + t) * LS + r] = sum;
        if (RIDE && extra) {
            const float sum2 = wave_sum(b0 + b1);
            if (lane == 0) ws.logits[(size_t)(t0 + t) * LS + d.E] = sum2;
        }
    }
}

// Selection + grouping as a launch of its own (many tokens): one token per wave, sixteen per
// workgroup; the workgroup that finishes last groups the pairs.
__global__ __launch_bounds__(1024) void moe_select_group_kernel(MoeWs ws, qkk_sel* __restrict__ sel, MoeDims d,
                                                                uint32_t N)
{
    __shared__ float s_log[16 * LOG_AREA];
    __shared__ uint32_t s_cnt[QKK_MAX_EXPERTS + 1], s_cur[QKK_MAX_EXPERTS + 1];
    __shared__ uint32_t s_last;
    const int wave = threadIdx.x >> 6;
    select_tokens<1>(ws, sel, d, N, blockIdx.x * 16 + wave, gridDim.x * 16, s_log + (size_t)wave * LOG_AREA, nullptr, true);
    __syncthreads();
    if (threadIdx.x == 0) s_last = arrive_last(&ws.counter[0], gridDim.x) ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        group_pairs_wg<16>(ws, sel, nullptr, d, N, s_cnt, s_cur);
        if (threadIdx.x == 0) ws.counter[0] = 0u;
    }
}

void moe_mfma_launch_shared(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                            const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st);
bool moe_rows_covers(const qkk_moe_layer* L, const MoeDims& d); // qk_moe_rows.hip
void moe_rows_launch_routed(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws, const MoeDims& d,
                            uint32_t N, uint32_t stages, hipStream_t st);
void moe_mfma_launch_routed(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                            const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st);
void moe_mfma_launch_fold(float* Y, const qkk_sel* sel, const MoeWs& ws, const MoeDims& d, uint32_t N, hipStream_t st);
void moe_mfma_launch_fold_norm(const float* resid, const float* w_next, float eps, float* S, float* Xn,
                               const qkk_sel* sel, const MoeWs& ws, const MoeDims& d, uint32_t N, hipStream_t st);
void moe_mfma_launch_fused(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws,
                           const MoeDims& d, uint32_t N, uint32_t stages, hipStream_t st);
constexpr uint32_t FUSED_MAX_ROWS = 32; // up to here the shared expert rides in the routed experts' launches

// The shared expert's chain runs on a side stream of the library, forked from and joined back into
// the caller's stream with events (capturable: under stream capture the side stream joins the
// caller's graph).  One side stream and one event pair PER CALLER STREAM and device, created under a
// lock on first use and kept until the process ends, default priority: two engines, or two host
// threads on streams of their own, never re-record each other's events.
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
};
static SideStream* side_stream(hipStream_t caller)
{
    static std::mutex lock;
    static std::map<std::pair<int, hipStream_t>, SideStream> made;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> hold(lock);
    auto it = made.find({dev, caller});
    if (it != made.end()) return &it->second;   // std::map: the address of an entry stays put
    SideStream s;
    if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess) return nullptr;
    if (hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
        if (s.fork) (void)hipEventDestroy(s.fork);
        (void)hipStreamDestroy(s.stream);
        return nullptr;
    }
    return &(made[{dev, caller}] = s);
}

// Reads (and clears) the current device's flag; the caller has synchronised the stream it asks about.
int moe_ws_alarm_take(bool* was_set)
{
    uint32_t* flag = nullptr;
    uint32_t v = 0;
    const uint32_t zero = 0;
    if (hipGetSymbolAddress((void**)&flag, HIP_SYMBOL(g_ws_alarm)) != hipSuccess || !flag ||
        hipMemcpy(&v, flag, sizeof v, hipMemcpyDeviceToHost) != hipSuccess ||
        (v && hipMemcpy(flag, &zero, sizeof zero, hipMemcpyHostToDevice) != hipSuccess)) {
        (void)hipGetLastError();
        return fail(QKK_EDEVICE, "moe: cannot read the workspace flag");
    }
    *was_set = v != 0;
    return QKK_OK;
}

// Host entry of the path for N >= 2 rows (arguments already validated).
int moe_grouped_launch(const qkk_moe_layer* L, const float* X, float* Y, qkk_sel* sel, void* workspace,
                       uint32_t N, uint32_t stages, hipStream_t st, const MoeTail* tail)
{
    const MoeDims d{L->n_embd, L->n_ff, L->n_expert, L->n_used};
    // the matrix-core kernels split n_embd over the eight waves of a workgroup, 256 weights each
    if (d.H != 2048) return fail(QKK_ESHAPE, "moe: several rows need n_embd = 2048 (got %u)", d.H);
    const MoeWs ws = ws_carve(workspace, d, N);
    const uint32_t experts_stages = stages & (QKK_STAGE_GATEUP | QKK_STAGE_DOWN);
    // the "moe_rows" switch: the routed experts through the row-split kernels (qk_moe_rows.hip); the shared expert
    // then always takes its own launches
    const bool rows = options().moe_rows != 0 && moe_rows_covers(L, d);
    const bool split = N > FUSED_MAX_ROWS || rows;
    // fork: the shared expert needs only X (and its own h), so it starts right away
    SideStream* side = experts_stages && split ? side_stream(st) : nullptr;
    if (experts_stages && split) {
        if (side && hipEventRecord(side->fork, st) == hipSuccess && hipStreamWaitEvent(side->stream, side->fork, 0) == hipSuccess)
            moe_mfma_launch_shared(L, X, sel, ws, d, N, stages, side->stream);
        else {
            side = nullptr; // no side stream: same work, in line
            moe_mfma_launch_shared(L, X, sel, ws, d, N, stages, st);
        }
    }
    if (stages & QKK_STAGE_ROUTE) {
        if (N <= SELECT_INLINE_MAX) { // logits, and selection + grouping in the last workgroup
            const uint32_t tasks = (d.E + 1) * ((N + 3) / 4);
            hipLaunchKernelGGL(moe_route_multi_kernel<8>, dim3((tasks + 7) / 8), dim3(512), 0, st, L->gate_inp,
                               L->gate_inp_shexp, X, ws, sel, d, N, 1u);
        } else { // tiled logits, then selection one token per wave + grouping
            constexpr uint32_t lds = LOGITS_TILE_TOKENS * 2048 * sizeof(float);
            static bool once = ((void)hipFuncSetAttribute((const void*)moe_logits_tiled_kernel<false>,
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                                (void)hipFuncSetAttribute((const void*)moe_logits_tiled_kernel<true>,
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), true);
            (void)once;
            const uint32_t tiles = (N + LOGITS_TILE_TOKENS - 1) / LOGITS_TILE_TOKENS, cus = persistent_blocks() / 4;
            const uint32_t g_all = (d.E + 1 + 7) / 8 * tiles, g_ride = (d.E + 7) / 8 * tiles;
            // fewer rounds of workgroups (one per CU: the activation tile takes 128 KB of LDS) decide
            const uint32_t ride = (g_ride + cus - 1) / cus < (g_all + cus - 1) / cus ? 1u : 0u;
            if (ride)
                hipLaunchKernelGGL(moe_logits_tiled_kernel<true>, dim3(g_ride), dim3(512), lds, st, L->gate_inp,
                                   L->gate_inp_shexp, X, ws, d, N);
            else
                hipLaunchKernelGGL(moe_logits_tiled_kernel<false>, dim3(g_all), dim3(512), lds, st, L->gate_inp,
                                   L->gate_inp_shexp, X, ws, d, N);
            hipLaunchKernelGGL(moe_select_group_kernel, dim3((N + 15) / 16), dim3(1024), 0, st, ws, sel, d, N);
        }
    }
    if (experts_stages) {
        if (rows) moe_rows_launch_routed(L, X, sel, ws, d, N, stages, st);
        else if (split) moe_mfma_launch_routed(L, X, sel, ws, d, N, stages, st);
        else moe_mfma_launch_fused(L, X, sel, ws, d, N, stages, st);
    }
    if (side) { // join
        if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess)
            return fail(QKK_EDEVICE, "moe: joining the shared-expert stream failed");
    }
    if (stages & QKK_STAGE_DOWN) {
        if (tail) moe_mfma_launch_fold_norm(tail->resid, tail->w_next, tail->eps, tail->S, tail->Xn, sel, ws, d, N, st);
        else moe_mfma_launch_fold(Y, sel, ws, d, N, st);
    }
    return check_launch("moe grouped path");
}

} // namespace qk
