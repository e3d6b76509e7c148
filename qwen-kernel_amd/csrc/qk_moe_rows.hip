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
// Work item = (active expert, 1, 2 or 4 consecutive blocks of 128 rows); its pair tiles of 16 follow one another,
// and within a tile the K steps of all its blocks are one pipeline (rows_stream, qk_rows.h).
// Behind the "moe_rows" switch until it has been run and timed on a device; the shared expert keeps the
// kernels of qk_moe_mfma.hip (it is one dense expert for every token).
// (reference shaders/moe_gateup_iq3_grouped_coopmat.comp:46-217, moe_down_iq4_grouped_coopmat.comp:45-166.)
#include "qk_moe_common.h"
#include "qk_rows.h"

#include <algorithm>

namespace qk {

// GATEUP: W0 = gate_exps, W1 = up_exps (IQ3_XXS rows of n_embd), activations X [N][n_embd], outputs h.
// else:   W0 = down_exps (rows of n_ff), activations h [N][k+1][n_ff], outputs contrib, weighted by the router.
template <int TYPE, bool GATEUP>
__global__ __launch_bounds__(MR_THREADS, 4) void moe_rows_kernel(const uint8_t* __restrict__ W0, const uint8_t* __restrict__ W1,
                                                                 const float* __restrict__ X, MoeWs ws,
                                                                 const qkk_sel* __restrict__ sel, MoeDims d, uint32_t N, uint32_t bpi)
{
    constexpr int NT = GATEUP ? 2 : 1;
    using G = RowsGeo<TYPE, NT>;
    QK_DYN_LDS(uint8_t, smem);
    __shared__ MfmaTables tab;
    __shared__ uint32_t s_tok[16], s_slot[16];
    __shared__ float s_wt[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, g = lane >> 4;
    fill_mfma_tables_for<TYPE>(tab, tid, MR_THREADS); // in place before the first barrier below
    const uint32_t K = GATEUP ? d.H : d.F, R = GATEUP ? d.F : d.H; // weights per row, rows per expert
    const uint32_t nfrag = K / 256, blocks_per_expert = R / MR_ROWS;
    const size_t stride = (size_t)nfrag * G::FB;                       // bytes of a weight row
    const size_t last_piece = (size_t)d.E * R * stride - 16;           // the tensors end on 16-byte boundaries (E * R * stride: R is a multiple of 128)
    const uint32_t n_active = active_count(ws, d);

    const uint32_t groups = blocks_per_expert / bpi; // a work item: bpi consecutive blocks of an active expert

    for (uint32_t item = blockIdx.x; item < n_active * groups; item += gridDim.x) {
        const ActiveExpert ae = active_expert(ws, item / groups, d, N);
        const uint32_t row0 = (item % groups) * bpi * MR_ROWS;
        const size_t base = ((size_t)ae.expert * R + row0) * stride; // the item's first row, both tensors

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
            const float* arow = GATEUP ? X + (size_t)s_tok[j] * d.H : ws.h + ((size_t)s_tok[j] * (d.k + 1) + s_slot[j]) * d.F;
            rows_stream<TYPE, NT>(
                W0, W1, bpi, [&](uint32_t b) { return base + (size_t)b * MR_ROWS * stride; }, stride, last_piece, nfrag, arow, smem,
                tab, tid, [&](uint32_t b, const float4v(&acc)[NT]) {
                    // D[4 g + e][j]: pair 4 g + e of the tile, row 16 wave + j of block b
                    const uint32_t row = row0 + b * MR_ROWS + 16 * wave + j;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t r = 4 * g + e;
                        if (r < np) {
                            const size_t rec = (size_t)s_tok[r] * (d.k + 1) + s_slot[r];
                            if constexpr (GATEUP) ws.h[rec * d.F + row] = (acc[0][e] / (1.f + expf(-acc[0][e]))) * acc[NT - 1][e];
                            else ws.contrib[rec * d.H + row] = s_wt[r] * acc[0][e];
                        }
                    }
                });
        }
    }
}

template <int TYPE, bool GATEUP>
static void launch_rows(const uint8_t* W0, const uint8_t* W1, const float* X, const MoeWs& ws, const qkk_sel* sel,
                        const MoeDims& d, uint32_t N, uint32_t experts, hipStream_t st)
{
    using G = RowsGeo<TYPE, GATEUP ? 2 : 1>;
    static const bool raised = ((void)hipFuncSetAttribute((const void*)moe_rows_kernel<TYPE, GATEUP>,
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)G::LDS_BYTES), true);
    (void)raised;
    // Work items of 4, 2 or 1 consecutive blocks of an expert: as long as there are items for every resident
    // workgroup (two per CU), fewer and longer ones -- the wait for the first fragments is paid once per item.
    // `experts` is an upper bound, the active ones are known on the device only.
    const uint32_t per_expert = (GATEUP ? d.F : d.H) / MR_ROWS, slots = persistent_blocks() / 2;
    uint32_t bpi = 4;
    while (bpi > 1 && (per_expert % bpi || experts * (per_expert / bpi) < slots)) bpi /= 2;
    const uint32_t blocks = std::max(1u, std::min(experts * (per_expert / bpi), slots));
    hipLaunchKernelGGL((moe_rows_kernel<TYPE, GATEUP>), dim3(blocks), dim3(MR_THREADS), G::LDS_BYTES, st, W0, W1, X, ws, sel, d, N, bpi);
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
