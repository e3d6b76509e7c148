// qk_rows.h -- a tile of 16 activation rows against a block of 128 weight rows (or 128 rows each of two
// tensors), with the eight waves of a workgroup splitting the weight ROWS: a wave owns 16 rows for all of K,
// so its accumulators are its outputs.  The activation operand of the 16 rows lives in LDS in operand order,
// converted to hi + lo halves once per workgroup and K step of 256 weights and read by every wave; the rows'
// fragments of a K step reach LDS as the aligned 16-byte pieces that cover them, the next step's pieces and
// activations in flight in registers during the arithmetic, from one block of rows into the next.  Decoder: BFrag<TYPE>::step, the cooperative
// stream's (qk_coop.h), so the same exactness (activations hi + lo, weights hi (+ lo)).
// Users: the routed experts' projections (qk_moe_rows.hip), the LM head for 2..16 rows (qk_head.hip).
#pragma once
#include "qk_coop.h"

namespace qk {

constexpr uint32_t MR_THREADS = 512, MR_ROWS = 128; // threads of a workgroup; weight rows of a work item

template <int TYPE, int NT>
struct RowsGeo {
    using F = BFrag<TYPE>;
    static constexpr uint32_t FB = F::BYTES;                             // bytes of a row's 256-weight fragment
    static constexpr uint32_t NPW = (FB + 15 + 15) / 16, WIN = NPW * 16; // pieces / bytes of a row's window
    static constexpr uint32_t SLOTS = NT * MR_ROWS;                      // row fragments of a K step in LDS
    static constexpr uint32_t PIECES = SLOTS * NPW;
    static constexpr int NLD = (PIECES + MR_THREADS - 1) / MR_THREADS;
    static constexpr uint32_t W_BYTES = SLOTS * WIN + 16, A_BYTES = 8 * 2 * 64 * 16; // one K step each
    static constexpr uint32_t LDS_BYTES = W_BYTES + 2 * A_BYTES;
};

// For each of `nblk` blocks of 128 weight rows in turn: acc[t][e] = sum over K of (row 16 wave + j of the block in
// tensor t: w0, and with NT = 2 also w1) . (activation row 4 g + e), lane = 16 g + j, handed to done(b, acc).  base_of(b): byte offset of block
// b's first row in every tensor (rows `stride` bytes apart, nfrag fragments each); reads are clamped to the
// 16-byte piece at `last_piece`, the tensors' last one.  arow: the activation row of THIS thread's lane j (thread
// (wave, lane) converts the operand of lane `lane` for instruction `wave` of a K step).  The K steps of all blocks
// form ONE pipeline: the first fragments of block b + 1 are in flight during the last step of block b, so the
// wait for memory at the head is paid once per call, not once per block.  With nfrag <= 2 the activation operand
// of every K step fits the two buffers and is converted once per call.
// smem: RowsGeo::LDS_BYTES; the caller has a barrier between the previous user of smem and this call, and one
// between this call and the next user.
template <int TYPE, int NT, class BaseOf, class Done>
__device__ __forceinline__ void rows_stream(const uint8_t* w0, const uint8_t* w1, uint32_t nblk, BaseOf base_of, size_t stride,
                                            size_t last_piece, uint32_t nfrag, const float* arow, uint8_t* smem,
                                            const MfmaTables& tab, int tid, Done done)
{
    using G = RowsGeo<TYPE, NT>;
    using F = typename G::F;
    constexpr uint32_t FB = G::FB, NPW = G::NPW, WIN = G::WIN, PIECES = G::PIECES;
    constexpr int NLD = G::NLD;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    uint8_t* s_w = smem;              // [SLOTS][WIN]
    uint8_t* s_a = smem + G::W_BYTES; // [2][step 8][hi, lo][lane 64] half8
    const int lane = tid & 63, wave = tid >> 6, j = lane & 15, g = lane >> 4;

    // piece p of a K step: row slot p / NPW (the first tensor's rows, then the second's), piece p % NPW of its
    // window.  Addresses are formed anew at every use (the thread index passes through an opaque register, or
    // the compiler forms the row offsets once per kernel and keeps them): four of them kept per thread across
    // the arithmetic cost more registers than the dozen integer operations they take.
    u32x4 ld[NLD];
    const auto fetch = [&](uint32_t b, uint32_t f) {
        uint32_t me = (uint32_t)tid;
        asm volatile("" : QK_REG(me));
        const size_t base = base_of(b);
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            const uint32_t p = min(me + MR_THREADS * n, PIECES - 1);
            const uint32_t slot = p / NPW, q = p % NPW;
            const uint8_t* t = NT > 1 && slot >= MR_ROWS ? w1 : w0; // a choice between two kernel arguments: the loads stay global loads
            const size_t at = base + (size_t)(slot % MR_ROWS) * stride + (size_t)f * FB; // the row's fragment f
            ld[n] = *(const u32x4*)(t + min((at & ~(size_t)15) + 16u * q, last_piece)); // its window starts at the 16-byte boundary below
        }
    };
    const auto commit = [&]() {
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            const uint32_t p = tid + MR_THREADS * n;
            if (PIECES % MR_THREADS == 0 || n + 1 < NLD || p < PIECES) *(u32x4*)(s_w + (p / NPW) * WIN + (p % NPW) * 16) = ld[n];
        }
    };
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
    const bool a_stays = nfrag <= 2; // step s reads buffer s & 1 = fragment s % nfrag for every block: filled by steps 0 and 1
    fetch(0, 0);
    load_a(0);
    commit();
    commit_a(0);
    __syncthreads();

    float4v acc[NT];
    const uint32_t steps = nblk * nfrag;
    uint32_t b = 0, f = 0; // block and fragment of step s
#pragma unroll 1
    for (uint32_t s = 0; s < steps; s++) {
        const uint32_t buf = s & 1u;
        const bool more = s + 1 < steps;                  // workgroup-uniform
        const bool wrap = f + 1 == nfrag;                 // this step closes its block
        const uint32_t nb = wrap ? b + 1 : b, nf = wrap ? 0u : f + 1;
        const bool conv = more && !(a_stays && s + 1 >= 2); // the next step's activations still have to be converted
        if (more) fetch(nb, nf);
        if (conv) load_a(nf);
        if (f == 0) {
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
        }
        // this lane's weight rows: row 16 wave + j of the block, in every tensor.  The tensors' tiles go through a
        // matrix-instruction step side by side: the activation operand of the step is read from LDS once for
        // both (its 2 KB per wave and step are the largest share of the workgroup's LDS traffic)
        const uint32_t skew = (uint32_t)((base_of(b) + (size_t)(16 * wave + j) * stride + (size_t)f * FB) & 15);
        const half8* ap = (const half8*)(s_a + buf * G::A_BYTES) + lane;
        F w[NT];
        float4v part[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            w[t].load(s_w + (size_t)(t * MR_ROWS + 16 * wave + j) * WIN + skew, 0, g);
            part[t] = float4v{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8 ahi = ap[(size_t)(i * 2) * 64], alo = ap[(size_t)(i * 2 + 1) * 64];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                half8 bl;
                const half8 bh = w[t].step(i, g, tab, bl);
                part[t] = mfma16x32(ahi, bh, part[t]);
                part[t] = mfma16x32(alo, bh, part[t]);
                if constexpr (F::SPLIT) part[t] = mfma16x32(ahi, bl, part[t]);
            }
            __builtin_amdgcn_sched_barrier(0); // keep the decode of later steps from piling up in registers
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const float sc = w[t].post();
            acc[t] += float4v{sc * part[t][0], sc * part[t][1], sc * part[t][2], sc * part[t][3]};
        }
        if (wrap) done(b, acc);
        if (more) {
            __syncthreads(); // every wave has read this step's rows
            commit();
            if (conv) commit_a(buf ^ 1u);
            __syncthreads(); // the next step's rows and activations are in place
        }
        b = nb;
        f = nf;
    }
}

} // namespace qk
