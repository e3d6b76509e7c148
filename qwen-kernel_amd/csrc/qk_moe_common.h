// qk_moe_common.h -- pieces shared by the single-slot and the grouped MoE paths: dimensions,
// workspace carving, the wave-level top-k selector.
#pragma once
#include "qk_device.h"
#include "qk_host.h"

namespace qk {

struct MoeDims {
    uint32_t H, F, E, k;
};

// Workspace layout (floats unless noted), per slot s:
//   logits  [E + 1]  (entry E = shared gate dot), stride LSTRIDE
//   h       [(k + 1) * F]
//   counter u32 (one per slot), after everything else
__host__ __device__ inline uint32_t lstride(uint32_t E) { return (E + 1 + 63) & ~63u; }

// One record per expert that at least one token picked: where its pairs are.
struct ActiveExpert {
    uint32_t expert, first, count, pad;
};

struct MoeWs {
    uint32_t* counter;    // [64] arrival counters; [0] is zero between steps
    float* logits;        // [n][lstride(E)]
    float* h;             // [n][k+1][F]
    // grouped path only (n >= 2)
    uint32_t* n_active;   // [1] (+3 pad)
    ActiveExpert* active; // [E]
    uint32_t* offsets;    // [E+1]
    uint32_t* pairs;      // [n*k] (token<<4)|pick
    float* contrib;       // [n][k+1][H], slot k = shared expert
};

// Layer tail behind the step: S = resid + (routed + shared), Xn = S * scale(S) * w_next.
struct MoeTail {
    const float* resid;
    const float* w_next;
    float eps;
    float* S;
    float* Xn;
};

// One row with the RMS norm in front (weights w) and the residual behind.
struct MoeNorm {
    const float* w;
    float eps;
    const float* mix = nullptr; // the row is X + mix ...
    float* sum = nullptr;       // ... which launch 1 stores here for launches 2 and 3
};

// The per-lane form of the one-row launches (qk_moe_lane.hip): launches 1 and 2, and launch 3.
void lane_route_gateup(const qkk_moe_layer* L, const float* X, const MoeWs& ws, qkk_sel* sel, const MoeDims& d,
                       uint32_t stages, const MoeNorm* norm, uint32_t rows, hipStream_t st);
void lane_down(const qkk_moe_layer* L, const MoeWs& ws, const qkk_sel* sel, float* Y, const MoeDims& d,
               const float* resid, uint32_t rows, hipStream_t st);

static inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static inline size_t ws_bytes(const MoeDims& d, uint32_t n)
{
    size_t b = 256 + align256((size_t)n * lstride(d.E) * 4) + align256((size_t)n * (d.k + 1) * d.F * 4);
    if (n >= 2)
        b += 256 + align256((size_t)d.E * sizeof(ActiveExpert)) + align256((size_t)(d.E + 1) * 4) +
             align256((size_t)n * d.k * 4) + align256((size_t)n * (d.k + 1) * d.H * 4);
    return b;
}

static inline MoeWs ws_carve(void* ws, const MoeDims& d, uint32_t n)
{
    MoeWs w;
    uint8_t* p = (uint8_t*)ws;
    w.counter = (uint32_t*)p; p += 256;
    w.logits = (float*)p; p += align256((size_t)n * lstride(d.E) * 4);
    w.h = (float*)p; p += align256((size_t)n * (d.k + 1) * d.F * 4);
    w.n_active = (uint32_t*)p; p += 256;
    w.active = (ActiveExpert*)p; p += align256((size_t)d.E * sizeof(ActiveExpert));
    w.offsets = (uint32_t*)p; p += align256((size_t)(d.E + 1) * 4);
    w.pairs = (uint32_t*)p; p += align256((size_t)n * d.k * 4);
    w.contrib = (float*)p;
    return w;
}

// ---- what the grouping left in the workspace, bounded by the shapes ------------------------------
// The expert kernels index tensors with these words.  A workspace that holds something else (first
// 256 bytes never cleared, a gate/up or down stage run before any routing, another stream still
// writing it) must give wrong numbers, never an access outside the tensors: every word is clamped
// to its range on the way in.
__device__ __forceinline__ uint32_t active_count(const MoeWs& ws, const MoeDims& d) { return min(*ws.n_active, d.E); }

__device__ __forceinline__ ActiveExpert active_expert(const MoeWs& ws, uint32_t w, const MoeDims& d, uint32_t N)
{
    ActiveExpert a = ws.active[w]; // w < active_count() <= E
    const uint32_t np = N * d.k;
    a.expert = min(a.expert, d.E - 1);
    a.first = min(a.first, np);
    a.count = min(a.count, np - a.first);
    return a;
}

// pair p of ws.pairs -> (token, pick)
__device__ __forceinline__ void pair_at(const MoeWs& ws, uint32_t p, const MoeDims& d, uint32_t N, uint32_t& tok,
                                        uint32_t& slot)
{
    const uint32_t pr = ws.pairs[p];
    tok = min(pr >> 4, N - 1);
    slot = min(pr & 15u, d.k - 1);
}

// ---- selector --------------------------------------------------------------------------
// One wave; lane L owns logits L, L+64, ... (NR register slots cover 64*NR experts).  Picks n_used
// times the maximum, lower id on ties; non-finite logits count as -3.4e38; weights exp(l - l0) over
// the picks, summed in pick order (reference shaders/moe_select.comp:28-34, 53-76).
// The loop is a chain of dependent wave-wide steps, so it is kept short: the exponentials are taken
// after it, by the lanes in parallel, and a tie for the maximum -- the only case that needs a second
// wave-wide reduction -- is detected with a ballot.
// Order-preserving map from non-NaN floats to signed ints (and back): the loop below compares,
// maximises and matches integers, which lets every reduction step be one DPP instruction.
__device__ __forceinline__ int32_t float_key(float f)
{
    const int32_t b = __builtin_bit_cast(int32_t, f + 0.f); // -0 -> +0: equal logits must tie
    return b ^ ((b >> 31) & 0x7FFFFFFF);
}
__device__ __forceinline__ float key_float(int32_t k)
{
    return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7FFFFFFF));
}

// Maximum over the wave, wave-uniform.
__device__ __forceinline__ int32_t wave_max_i32(int32_t x)
{
    x = max(x, dpp_i<DPP_XOR1>(x));
    x = max(x, dpp_i<DPP_XOR2>(x));
    x = max(x, dpp_i<DPP_HALF_MIRROR>(x));
    x = max(x, dpp_i<DPP_MIRROR>(x));
    const int32_t a = max(__builtin_amdgcn_readlane(x, 0), __builtin_amdgcn_readlane(x, 16));
    const int32_t b = max(__builtin_amdgcn_readlane(x, 32), __builtin_amdgcn_readlane(x, 48));
    return max(a, b);
}

template <int NR>
__device__ static inline void select_wave_n(const float* __restrict__ logits, uint32_t E, uint32_t k,
                                            qkk_sel* __restrict__ out, uint32_t* ids_copy)
{
    constexpr float FLOOR = -3.4e38f;
    const int lane = threadIdx.x & 63;
    int32_t v[NR];
#pragma unroll
    for (int i = 0; i < NR; i++) {
        const uint32_t e = lane + 64 * i;
        float l = e < E ? logits[e] : FLOOR;
        if (isnan(l) || isinf(l)) l = FLOOR;
        v[i] = float_key(l);
    }
    const int32_t floor_key = float_key(FLOOR);
    int32_t top = 0, mym = 0;
    uint32_t myid = 0;
    for (uint32_t r = 0; r < k; r++) {
        int32_t bv = v[0];
        uint32_t bi = lane;
#pragma unroll
        for (int i = 1; i < NR; i++)
            if (v[i] > bv) { bv = v[i]; bi = lane + 64 * i; }
        const int32_t m = wave_max_i32(bv);
        const uint64_t tie = __builtin_amdgcn_ballot_w64(bv == m); // never empty: m is some lane's bv
        uint32_t id;
        if (__builtin_popcountll(tie) == 1) // wave-uniform
            id = (uint32_t)__builtin_amdgcn_readlane((int)bi, __builtin_ctzll(tie));
        else
            id = wave_min_u32(bv == m ? bi : 0x7FFFFFFFu);
        // retire the winner
#pragma unroll
        for (int i = 0; i < NR; i++)
            if ((uint32_t)(lane + 64 * i) == id) v[i] = floor_key;
        if (r == 0) top = m;
        if ((uint32_t)lane == r) { mym = m; myid = min(id, E - 1); }
    }
    const float p = (uint32_t)lane < k ? expf(key_float(mym) - key_float(top)) : 0.f;
    float wsum = 0.f;
    for (uint32_t r = 0; r < k; r++) wsum += readlane_f(p, (int)r); // pick order
    if ((uint32_t)lane < k) {
        out->ids[lane] = myid;
        out->w[lane] = p / wsum;
        if (ids_copy) ids_copy[lane] = myid; // for a grouping pass in the same workgroup (LDS)
    }
}

__device__ static inline void select_wave(const float* __restrict__ logits, uint32_t E, uint32_t k,
                                          qkk_sel* __restrict__ out, uint32_t* ids_copy = nullptr)
{
    if (E <= 256) select_wave_n<4>(logits, E, k, out, ids_copy);
    else select_wave_n<QKK_MAX_EXPERTS / 64>(logits, E, k, out, ids_copy);
}

// ---- the same selection by a whole workgroup of four waves, without a chain of dependent rounds ------
// The one-wave selector above is n_used rounds, each a chain of dependent cross-lane steps (about 1.7 us
// for 8 of 256 on a lone wave).  Here every element finds its RANK by counting, and counting is a stream of
// independent compares.  An element is (logit key, expert id) packed into 64 bits so that "greater" is
// "picked earlier" (higher logit first, lower id on equal logits: a strict total order).  Thread t holds the
// experts t and t + 256; a wave ranks its up to 128 elements among themselves (the others' values come as
// LDS broadcasts), the n_used best of each wave -- a global pick is always among its own wave's best n_used --
// are ranked again by wave 0 among the 4 * n_used candidates, and a candidate's rank there is its pick
// number.  The reference's degenerate case (fewer finite logits than picks: once they are used up every
// further round finds all entries at the floor and takes entry 0, shaders/moe_select.comp:53-70) is
// reproduced from the count of finite logits.  Same ids, same weights as select_wave.
struct SelectScratch {
    uint64_t elem[QKK_MAX_EXPERTS];
    uint64_t cand[4 * QKK_MAX_USED];
    float logit[QKK_MAX_USED];
    uint32_t finite[4];
};

// l0 / l1: this thread's logits of experts threadIdx.x and threadIdx.x + 256 (ignored where the id is not
// below E); shared_logit: the shared gate's logit (thread 0).  All 256 threads call; `out` (LDS) is complete
// after the caller's next workgroup barrier.
__device__ static inline void select_block(float l0, float l1, float shared_logit, uint32_t E, uint32_t k,
                                           qkk_sel* __restrict__ out, SelectScratch& sc)
{
    constexpr float FLOOR = -3.4e38f;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t floor_hi = (uint32_t)float_key(FLOOR) ^ 0x80000000u;
    const auto pack = [&](float l, uint32_t id) -> uint64_t {
        if (id >= E || isnan(l) || isinf(l)) l = FLOOR;
        return ((uint64_t)((uint32_t)float_key(l) ^ 0x80000000u) << 32) | (uint32_t)~id;
    };
    const bool wide = E > 256; // workgroup-uniform
    const uint64_t c0 = pack(l0, tid), c1 = pack(l1, tid + 256);
    sc.elem[tid] = c0;
    sc.elem[256 + tid] = c1;
    const uint32_t nf = __builtin_popcountll(__builtin_amdgcn_ballot_w64((uint32_t)(c0 >> 32) > floor_hi)) +
                        __builtin_popcountll(__builtin_amdgcn_ballot_w64((uint32_t)(c1 >> 32) > floor_hi));
    if (lane == 0) sc.finite[wave] = nf;
    __syncthreads();
    // rank inside the wave
    uint32_t r0 = 0, r1 = 0;
#pragma unroll 16
    for (uint32_t jj = 0; jj < 64; jj++) {
        const uint64_t o = sc.elem[64 * wave + jj];
        r0 += o > c0;
        r1 += o > c1;
    }
    if (wide) {
#pragma unroll 16
        for (uint32_t jj = 0; jj < 64; jj++) {
            const uint64_t o = sc.elem[256 + 64 * wave + jj];
            r0 += o > c0;
            r1 += o > c1;
        }
        if (r1 < k) sc.cand[wave * k + r1] = c1;
    }
    if (r0 < k) sc.cand[wave * k + r0] = c0;
    __syncthreads();
    if (wave != 0) return;
    const uint32_t nc = 4 * k;
    const uint64_t mine = lane < nc ? sc.cand[lane] : 0;
    uint32_t rank = 0;
    for (uint32_t jj = 0; jj < nc; jj++) rank += sc.cand[jj] > mine;
    const uint32_t n_finite = min(sc.finite[0] + sc.finite[1] + sc.finite[2] + sc.finite[3], k);
    if (lane < nc && (uint32_t)(mine >> 32) > floor_hi && rank < k) {
        out->ids[rank] = min(~(uint32_t)mine, E - 1);
        sc.logit[rank] = key_float((int32_t)((uint32_t)(mine >> 32) ^ 0x80000000u));
    }
    if (lane >= n_finite && lane < k) { // the finite logits are used up: entry 0, at the floor
        out->ids[lane] = 0;
        sc.logit[lane] = FLOOR;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float p = lane < k ? expf(sc.logit[lane] - sc.logit[0]) : 0.f;
    float wsum = 0.f;
    for (uint32_t r = 0; r < k; r++) wsum += readlane_f(p, (int)r); // pick order
    if (lane < k) out->w[lane] = p / wsum;
    if (lane == 0) out->w_shared = 1.f / (1.f + expf(-shared_logit));
}

} // namespace qk
