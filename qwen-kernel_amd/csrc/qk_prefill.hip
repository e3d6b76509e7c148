// qk_prefill.hip -- batched-prefill kernels for gfx950: pair grouping, the Q8_0 dense
// projection GEMM and the grouped-expert MoE GEMMs (fp16 tiles dequantised in LDS, MFMA
// with fp32 accumulation).
#include "qk_device.h"
#include "qk_host.h"

namespace qk {

// Counting sort of (token, pick) pairs by expert in one workgroup.  Pairs inside an expert
// come out in ascending (token, pick) order: each thread owns a contiguous run of pairs, a
// prefix sum over per-thread counts replaces the reference's LDS atomics
// (reference shaders/moe_group_pairs.comp:29,48), so the output is deterministic.
__global__ __launch_bounds__(1024) void group_pairs_kernel(const qkk_sel* __restrict__ sel,
                                                           uint32_t n_tokens, uint32_t E, uint32_t k,
                                                           uint32_t* __restrict__ offsets,
                                                           uint32_t* __restrict__ pairs)
{
    __shared__ uint32_t s_count[QKK_MAX_EXPERTS + 1];
    __shared__ uint32_t s_base[QKK_MAX_EXPERTS + 1];
    const uint32_t np = n_tokens * k;
    for (uint32_t e = threadIdx.x; e <= E; e += blockDim.x) s_count[e] = 0;
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < np; p += blockDim.x)
        atomicAdd(&s_count[min(sel[p / k].ids[p % k], E - 1)], 1u);
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t off = 0;
        for (uint32_t e = 0; e < E; e++) {
            s_base[e] = off;
            off += s_count[e];
        }
        s_base[E] = off;
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = s_base[e];
    // one thread per expert walks the pairs in order: E <= 512 threads busy, np*E/blockDim
    // comparisons each -- small next to the GEMMs it feeds, and order-stable
    for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) {
        if (s_count[e] == 0) continue;
        uint32_t dst = s_base[e];
        for (uint32_t p = 0; p < np; p++)
            if (min(sel[p / k].ids[p % k], E - 1) == e) pairs[dst++] = ((p / k) << 4) | (p % k);
    }
}

} // namespace qk

using namespace qk;

extern "C" {

int qkk_moe_group_pairs(const qkk_sel* sel, uint32_t n_tokens, uint32_t n_expert, uint32_t n_used,
                        uint32_t* offsets, uint32_t* pairs, void* stream)
{
    if (!sel || !offsets || !pairs) return fail(QKK_EINVAL, "qkk_moe_group_pairs: null pointer");
    if (n_expert < 1 || n_expert > QKK_MAX_EXPERTS || n_used < 1 || n_used > QKK_MAX_USED)
        return fail(QKK_ESHAPE, "qkk_moe_group_pairs: n_expert %u / n_used %u out of range", n_expert, n_used);
    if (n_tokens == 0 || n_tokens > (1u << 28) / 16)
        return fail(QKK_ESHAPE, "qkk_moe_group_pairs: n_tokens %u out of range", n_tokens);
    if (int rc = require_device()) return rc;
    hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(1024), 0, as_stream(stream), sel, n_tokens, n_expert,
                       n_used, offsets, pairs);
    return check_launch("qkk_moe_group_pairs");
}

int qkk_gemm_q8_0(const void*, const float*, float*, uint32_t, uint32_t, uint32_t, void*)
{
    return fail(QKK_ESHAPE, "qkk_gemm_q8_0: not built yet");
}
size_t qkk_moe_prefill_workspace_bytes(const qkk_moe_layer*, uint32_t) { return 0; }
int qkk_moe_prefill(const qkk_moe_layer*, const float*, float*, qkk_sel*, void*, size_t, uint32_t, void*)
{
    return fail(QKK_ESHAPE, "qkk_moe_prefill: not built yet");
}

} // extern "C"
