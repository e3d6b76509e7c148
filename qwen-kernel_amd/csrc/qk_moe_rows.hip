// qk_moe_rows.hip -- the routed experts' gate/up and down projections for several tokens with the waves
// of a workgroup splitting the weight ROWS instead of K.
//
// The kernels of qk_moe_mfma.hip split K over the eight waves (each keeps its K slice of the 16 activation
// rows in registers), which costs, per 16 weight rows, partial results through LDS, a sum over the waves
// and a barrier: measured about 6 k clocks per batch around 0.8 k clocks of matrix instructions, and it is
// that fixed cost -- not memory, not decode -- that holds the 16-slot step and the 128-token prefill at a
// fifth of the memory roofline.  An expert seldom has more than a few tokens, so the activation operand of
// a whole tile of 16 (token, pick) pairs is small: 16 KB per 256 weights of K as hi + lo halves.  Here it
// lives in LDS, in operand order, converted once per workgroup and K step and read by every wave; a wave owns
// 16 weight rows (for gate/up: the same 16 rows of gate AND of up) for all of K, so its accumulators are its
// outputs -- no partial results, no sum across waves -- and SiLU(gate) * up is formed in registers.  The
// rows' fragments of a K step reach LDS as the aligned 16-byte pieces that cover them (as in
// qk_gemm_tiled.hip), the next step's pieces and activations in flight in registers during the arithmetic;
// 64 KB of LDS and under 128 registers per lane, so two workgroups share a CU.  Decoder: BFrag<TYPE>::step, the
// cooperative stream's, so the same exactness (activations hi + lo, weights hi (+ lo)).
// Work item = (active expert, block of 128 rows); its pair tiles of 16 follow one another.
// Behind the "moe_rows" switch until it has been run and timed on a device; the shared expert keeps the
// kernels of qk_moe_mfma.hip (it is one dense expert for every token).
// (reference shaders/moe_gateup_iq3_grouped_coopmat.comp:46-217, moe_down_iq4_grouped_coopmat.comp:45-166.)
#include "qk_coop.h"
#include "qk_moe_common.h"

#include <algorithm>

namespace qk {

constexpr uint32_t MR_THREADS = 512, MR_ROWS = 128; // threads of a workgroup; weight rows of a work item

template <int TYPE, bool GATEUP>
struct RowsGeo {
    using F = BFrag<TYPE>;
    static constexpr uint32_t FB = F::BYTES;                       // bytes of a row's 256-weight fragment
    static constexpr uint32_t NPW = (FB + 15 + 15) / 16, WIN = NPW * 16; // pieces / bytes of a row's window
    static constexpr uint32_t SLOTS = GATEUP ? 2 * MR_ROWS : MR_ROWS;    // row fragments of a K step in LDS
    static constexpr uint32_t PIECES = SLOTS * NPW;
    static constexpr int NLD = (PIECES + MR_THREADS - 1) / MR_THREADS;
    static constexpr uint32_t W_BYTES = SLOTS * WIN + 16, A_BYTES = 8 * 2 * 64 * 16; // one K step each
    static constexpr uint32_t LDS_BYTES = W_BYTES + 2 * A_BYTES;
};

// GATEUP: W0 = gate_exps, W1 = up_exps (IQ3_XXS rows of n_embd), activations X [N][n_embd], outputs h.
// else:   W0 = down_exps (rows of n_ff), activations h [N][k+1][n_ff], outputs contrib, weighted by the router.
template <int TYPE, bool GATEUP>
__global__ __launch_bounds__(MR_THREADS, 4) void moe_rows_kernel(const uint8_t* __restrict__ W0, const uint8_t* __restrict__ W1,
                                                                 const float* __restrict__ X, MoeWs ws,
                                                                 const qkk_sel* __restrict__ sel, MoeDims d, uint32_t N)
{
    using G = RowsGeo<TYPE, GATEUP>;
    using F = typename G::F;
    constexpr uint32_t FB = G::FB, NPW = G::NPW, WIN = G::WIN, PIECES = G::PIECES;
    constexpr int NLD = G::NLD, NT = GATEUP ? 2 : 1;
    QK_DYN_LDS(uint8_t, smem);
    uint8_t* s_w = smem;                 // [SLOTS][WIN]
    uint8_t* s_a = smem + G::W_BYTES;    // [2][step 8][hi, lo][lane 64] half8
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, g = lane >> 4;
    fill_mfma_tables_for<TYPE>(tab, tid, MR_THREADS); // in place before the first barrier below
    const uint32_t K = GATEUP ? d.H : d.F, R = GATEUP ? d.F : d.H; // weights per row, rows per expert
    const uint32_t nfrag = K / 256, blocks_per_expert = R / MR_ROWS;
    const size_t stride = (size_t)nfrag * FB;                          // bytes of a weight row
    const size_t last_piece = (size_t)d.E * R * stride - 16;           // the tensors end on 16-byte boundaries (E * R * stride: R is a multiple of 128)
    const uint32_t n_active = active_count(ws, d);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

    for (uint32_t item = blockIdx.x; item < n_active * blocks_per_expert; item += gridDim.x) {
        const ActiveExpert ae = active_expert(ws, item / blocks_per_expert, d, N);
        const uint32_t row0 = (item % blocks_per_expert) * MR_ROWS;
        const size_t base = ((size_t)ae.expert * R + row0) * stride; // the block's first row, both tensors

        // piece p of a K step: row slot p / NPW (gate rows, then up rows), piece p % NPW of its window.  Addresses
        // are formed anew at every use (the thread index passes through an opaque register, or the compiler
        // forms the row offsets once per kernel and keeps them): four of them kept per thread across the
        // arithmetic cost more registers than the dozen integer operations they take.
        u32x4 ld[NLD];
        const auto fetch = [&](uint32_t f) {
            uint32_t me = (uint32_t)tid;
            asm volatile("" : QK_REG(me));
#pragma unroll
            for (int n = 0; n < NLD; n++) {
                const uint32_t p = min(me + MR_THREADS * n, PIECES - 1);
                const uint32_t slot = p / NPW, q = p % NPW;
                const uint8_t* tens = GATEUP && slot >= MR_ROWS ? W1 : W0;
                const size_t at = base + (size_t)(slot % MR_ROWS) * stride + (size_t)f * FB; // the row's fragment f
                ld[n] = *(const u32x4*)(tens + min((at & ~(size_t)15) + 16u * q, last_piece));   // its window starts at the 16-byte boundary below
            }
        };
        const auto commit = [&]() {
#pragma unroll
            for (int n = 0; n < NLD; n++) {
                const uint32_t p = tid + MR_THREADS * n;
                if (PIECES % MR_THREADS == 0 || n + 1 < NLD || p < PIECES) *(u32x4*)(s_w + (p / NPW) * WIN + (p % NPW) * 16) = ld[n];
            }
        };
        // this lane's weight rows: row 16 wave + j of the block (gate tile, and for gate/up the up tile)
        const size_t my_at = base + (size_t)(16 * wave + j) * stride;

        for (uint32_t t0 = 0; t0 < ae.count; t0 += 16) {
            const uint32_t np = min(16u, ae.count - t0);
            __syncthreads(); // the previous tile's LDS is consumed
            if (tid < 16) {
                uint32_t tok = 0, slot = 0;
                float wt = 0.f;
                pair_at(ws, ae.first + t0 + min((uint32_t)tid, np - 1), d, N, tok, slot); // pairs behind the tile repeat its last one
                if (!GATEUP) wt = sel[tok].w[slot];
                s_tok[tid] = tok; s_slot[tid] = slot; s_wt[tid] = wt;
            }
            __syncthreads();
            // thread (step i = wave, lane): the operand of lane (pair j, group g) for step i of a K step
            const float* arow = GATEUP ? X + (size_t)s_tok[j] * d.H : ws.h + ((size_t)s_tok[j] * (d.k + 1) + s_slot[j]) * d.F;
            const uint32_t acut = F::LAYOUT == 0 ? 64 * g + 8 * wave : 128 * (g >> 1) + 32 * (wave >> 1) + 16 * (g & 1) + 8 * (wave & 1);
            float4 ar[2];
            const auto load_a = [&](uint32_t f) {
                ar[0] = *(const float4*)(arow + 256 * f + acut);
                ar[1] = *(const float4*)(arow + 256 * f + acut + 4);
            };
            const auto commit_a = [&](uint32_t buf) {
                const float x[8] = {ar[0].x, ar[0].y, ar[0].z, ar[0].w, ar[1].x, ar[1].y, ar[1].z, ar[1].w};
                half8 hi, lo;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    hi[e] = (_Float16)x[e];
                    lo[e] = (_Float16)(x[e] - (float)hi[e]);
                }
                half8* dstp = (half8*)(s_a + buf * G::A_BYTES) + (size_t)(wave * 2) * 64 + lane;
                dstp[0] = hi;
                dstp[64] = lo;
            };
            fetch(0);
            load_a(0);
            commit();
            commit_a(0);
            __syncthreads();

            float4v acc[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
            for (uint32_t f = 0; f < nfrag; f++) {
                const uint32_t buf = f & 1u;
                const bool more = f + 1 < nfrag; // workgroup-uniform
                if (more) {
                    fetch(f + 1);
                    load_a(f + 1);
                }
                // one tile after the other (gate, then up): one set of fragment registers and decode temporaries
                // alive at a time; the waves of the SIMD fill each other's matrix-instruction latencies
                const half8* ap = (const half8*)(s_a + buf * G::A_BYTES) + lane;
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    asm volatile("" ::: "memory"); // the second tile reads its activation operands again rather than keeping the first's 64 registers
                    F w;
                    w.load(s_w + (size_t)(t * MR_ROWS + 16 * wave + j) * WIN + ((my_at + (size_t)f * FB) & 15), 0, g);
                    float4v part = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const half8 ahi = ap[(size_t)(i * 2) * 64], alo = ap[(size_t)(i * 2 + 1) * 64];
                        half8 bl;
                        const half8 bh = w.step(i, g, tab, bl);
                        part = mfma16x32(ahi, bh, part);
                        part = mfma16x32(alo, bh, part);
                        if constexpr (F::SPLIT) part = mfma16x32(ahi, bl, part);
                        __builtin_amdgcn_sched_barrier(0); // keep the decode of later steps from piling up in registers
                    }
                    const float sc = w.post();
                    acc[t] += float4v{sc * part[0], sc * part[1], sc * part[2], sc * part[3]};
                }
                if (more) {
                    __syncthreads(); // every wave has read this step's rows
                    commit();
                    commit_a(buf ^ 1u);
                    __syncthreads(); // the next step's rows and activations are in place
                }
            }
            // D[4 g + e][j]: pair 4 g + e of the tile, row 16 wave + j of the block
            const uint32_t row = row0 + 16 * wave + j;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t r = 4 * g + e;
                if (r < np) {
                    const size_t rec = (size_t)s_tok[r] * (d.k + 1) + s_slot[r];
                    if constexpr (GATEUP) ws.h[rec * d.F + row] = (acc[0][e] / (1.f + expf(-acc[0][e]))) * acc[NT - 1][e];
                    else ws.contrib[rec * d.H + row] = s_wt[r] * acc[0][e];
                }
            }
        }
    }
}

template <int TYPE, bool GATEUP>
static void launch_rows(const uint8_t* W0, const uint8_t* W1, const float* X, const MoeWs& ws, const qkk_sel* sel,
                        const MoeDims& d, uint32_t N, uint32_t experts, hipStream_t st)
{
    using G = RowsGeo<TYPE, GATEUP>;
    static const bool raised = ((void)hipFuncSetAttribute((const void*)moe_rows_kernel<TYPE, GATEUP>,
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)G::LDS_BYTES), true);
    (void)raised;
    const uint32_t items = experts * ((GATEUP ? d.F : d.H) / MR_ROWS); // an upper bound: the active experts are known on the device
    const uint32_t blocks = std::max(1u, std::min(items, 2 * (persistent_blocks() / 4)));
    hipLaunchKernelGGL((moe_rows_kernel<TYPE, GATEUP>), dim3(blocks), dim3(MR_THREADS), G::LDS_BYTES, st, W0, W1, X, ws, sel, d, N);
}

// Whether the row-split form covers the layer: whole K steps of 256 weights, whole blocks of 128 rows, the
// block formats instantiated below.
bool moe_rows_covers(const qkk_moe_layer* L, const MoeDims& d)
{
    return d.H % 256 == 0 && d.F % 256 == 0 && d.F % MR_ROWS == 0 && d.H % MR_ROWS == 0 && L->gu_type == QKK_IQ3_XXS &&
           (L->down_type == QKK_IQ4_XS || L->down_type == QKK_Q6_K);
}

// The routed experts' launches of a step in the row-split form (for a layer that moe_rows_covers).
void moe_rows_launch_routed(const qkk_moe_layer* L, const float* X, const qkk_sel* sel, const MoeWs& ws, const MoeDims& d,
                            uint32_t N, uint32_t stages, hipStream_t st)
{
    const uint32_t experts = (uint32_t)std::min<uint64_t>(d.E, (uint64_t)N * d.k);
    if (stages & QKK_STAGE_GATEUP)
        launch_rows<QKK_IQ3_XXS, true>((const uint8_t*)L->gate_exps, (const uint8_t*)L->up_exps, X, ws, sel, d, N, experts, st);
    if (stages & QKK_STAGE_DOWN) {
        if (L->down_type == QKK_IQ4_XS) launch_rows<QKK_IQ4_XS, false>((const uint8_t*)L->down_exps, nullptr, X, ws, sel, d, N, experts, st);
        else launch_rows<QKK_Q6_K, false>((const uint8_t*)L->down_exps, nullptr, X, ws, sel, d, N, experts, st);
    }
}

} // namespace qk
