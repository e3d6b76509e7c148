// Host-side stand-in for <hip/hip_runtime.h>: lets the HIP sources under qwen-kernel_amd/csrc compile
// as plain C++ and run on the CPU, one OS thread per GPU thread, so that their indexing can be
// checked against guard pages and their results against the oracle without a GPU.  TEST
// INFRASTRUCTURE ONLY: nothing in the product loads the library built from this; speed is irrelevant.
//
// Model: every GPU thread of a workgroup is a fiber on one OS thread (workgroups of a launch run on a
// few OS threads side by side, `__shared__` is thread-local storage); a fiber runs until it reaches a
// barrier that is not complete.  __syncthreads() is a real barrier; every cross-lane operation (DPP,
// readlane, bpermute, ballot, shuffles, MFMA) exchanges values through a per-wave buffer between two
// wave barriers, and __builtin_amdgcn_wave_barrier() is a real wave barrier -- code that relies on
// the lanes of a wave running in lockstep has to say so with one.  Lanes do NOT run in lockstep here:
// a lane runs ahead of the others of its wave up to the next barrier.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <functional>
#include <vector>
#include <type_traits>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static thread_local
#define __align__(n) __attribute__((aligned(n)))
// the kernels' hooks (qk_device.h): dynamic LDS comes from the launch, register pins become memory pins
#define QK_DYN_LDS(type, name) type* name = (type*)emu::dyn_lds()
#define QK_REG(x) "+m"(x)
// table lookups in LDS report this lane's address and width; the runtime models the banks (below)
#define QK_LDS_PROBE(site, ptr, bytes) do { if (emu::g_lds_probe_on) emu::lds_probe(site, ptr, bytes); } while (0)

struct uint2 { uint32_t x, y; };
struct __attribute__((aligned(16))) uint4 { uint32_t x, y, z, w; };
struct float2 { float x, y; };
struct __attribute__((aligned(16))) float4 { float x, y, z, w; };
struct dim3 {
    uint32_t x, y, z;
    dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef void* hipStream_t;
typedef void* hipEvent_t;
enum hipError_t { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorUnknown = 999 };
enum hipMemcpyKind { hipMemcpyHostToHost = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum hipStreamCaptureMode { hipStreamCaptureModeGlobal = 0, hipStreamCaptureModeThreadLocal = 1 };
enum { hipHostMallocDefault = 0 };
typedef struct emu_graph* hipGraph_t;
typedef struct emu_graph_exec* hipGraphExec_t;
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 16 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
enum { hipStreamNonBlocking = 1, hipEventDisableTiming = 2 };
struct hipDeviceProp_t { char gcnArchName[64]; int multiProcessorCount; };

namespace emu {
struct Idx { uint32_t x, y, z; };
const Idx& cur_thread();
const Idx& cur_block();
extern Idx g_block_dim, g_grid_dim;
void* dyn_lds();
void block_barrier();
void wave_barrier();
// every lane of the calling wave passes its value; returns the 64 values (valid until the next exchange)
const uint64_t* exchange(uint64_t v);
void exchange_done();
void run(dim3 grid, dim3 block, size_t lds, const std::function<void()>& body);
// LDS bank model for marked lookups (off unless a test switches it on): a wave instruction's addresses
// are gathered from its lanes, and it costs, pass by pass (64 lanes of 4 bytes, 32 of 8, 16 of 16), the
// largest number of distinct dwords that any of the 64 four-byte banks is asked for; a conflict-free
// pass costs 1.  A proxy for the device's LDS, not a measurement of it.
extern bool g_lds_probe_on;
void lds_probe(int site, const void* p, int bytes);
// Stream capture: between hipStreamBeginCapture and hipStreamEndCapture (per host thread) launches,
// copies and fills are recorded instead of run; a graph is the recorded list, a launch of it runs
// the list in order.  submit() runs `op` now, or records it while the calling thread captures.
void submit(std::function<void()> op);
bool capture_begin();
struct Graph { std::vector<std::function<void()>> ops; };
Graph* capture_end();
} // namespace emu

#define threadIdx emu::cur_thread()
#define blockIdx emu::cur_block()
#define blockDim emu::g_block_dim
#define gridDim emu::g_grid_dim

template <class K, class... A>
static inline void emu_launch(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t, A... args)
{
    emu::submit([=]() { emu::run(grid, block, lds, [=]() { kernel(args...); }); });
}
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) emu_launch(kernel, grid, block, lds, stream, __VA_ARGS__)
#define HIP_SYMBOL(x) ((const void*)&(x))

// ---- runtime API used by the launchers ----------------------------------------------------------
static inline hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
static inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "host build"; }
static inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 4; return hipSuccess; } // a small "device": 4 CUs
static inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
static inline hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) { snprintf(p->gcnArchName, 64, "host"); p->multiProcessorCount = 4; return hipSuccess; }
static inline hipError_t hipMemcpyAsync(void* d, const void* s, size_t n, hipMemcpyKind, hipStream_t) { emu::submit([=]() { memmove(d, s, n); }); return hipSuccess; }
static inline hipError_t hipGetSymbolAddress(void** p, const void* sym) { *p = (void*)sym; return hipSuccess; }
hipError_t hipMalloc(void** p, size_t n);   // ends at a guard page
hipError_t hipFree(void* p);
template <class T> static inline hipError_t hipMalloc(T** p, size_t n) { return hipMalloc((void**)p, n); }
static inline hipError_t hipHostMalloc(void** p, size_t n, unsigned = 0) { *p = malloc(n ? n : 1); return *p ? hipSuccess : hipErrorUnknown; }
template <class T> static inline hipError_t hipHostMalloc(T** p, size_t n, unsigned f = 0) { return hipHostMalloc((void**)p, n, f); }
static inline hipError_t hipHostFree(void* p) { free(p); return hipSuccess; }
static inline hipError_t hipMemcpy(void* d, const void* s, size_t n, hipMemcpyKind) { memmove(d, s, n); return hipSuccess; }
static inline hipError_t hipMemset(void* d, int v, size_t n) { memset(d, v, n); return hipSuccess; }
static inline hipError_t hipMemsetAsync(void* d, int v, size_t n, hipStream_t = nullptr) { emu::submit([=]() { memset(d, v, n); }); return hipSuccess; }
static inline hipError_t hipMemGetInfo(size_t* f, size_t* t)
{   // 64 GB free unless QK_EMU_FREE_BYTES says otherwise (for tests of the callers' checks)
    const char* e = getenv("QK_EMU_FREE_BYTES");
    *f = e ? (size_t)strtoull(e, nullptr, 10) : (size_t)64 << 30;
    *t = (size_t)64 << 30;
    return hipSuccess;
}
static inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
static inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
static inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
static inline hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }
template <class K> static inline hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int* n, K, int, size_t) { *n = 2; return hipSuccess; }
static inline hipError_t hipStreamBeginCapture(hipStream_t, hipStreamCaptureMode) { return emu::capture_begin() ? hipSuccess : hipErrorUnknown; }
static inline hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t* g) { *g = (hipGraph_t)emu::capture_end(); return *g ? hipSuccess : hipErrorUnknown; }
static inline hipError_t hipGraphInstantiate(hipGraphExec_t* e, hipGraph_t g, void*, void*, size_t)
{
    *e = g ? (hipGraphExec_t) new emu::Graph(*(emu::Graph*)g) : nullptr;
    return *e ? hipSuccess : hipErrorInvalidValue;
}
static inline hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t)
{
    if (!e) return hipErrorInvalidValue;
    for (const auto& op : ((emu::Graph*)e)->ops) emu::submit(op);
    return hipSuccess;
}
static inline hipError_t hipGraphDestroy(hipGraph_t g) { delete (emu::Graph*)g; return hipSuccess; }
static inline hipError_t hipGraphExecDestroy(hipGraphExec_t e) { delete (emu::Graph*)e; return hipSuccess; }
static inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = nullptr; return hipSuccess; }
static inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = nullptr; return hipSuccess; }
static inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
static inline hipError_t hipEventCreate(hipEvent_t* e) { *e = nullptr; return hipSuccess; }
static inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
static inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 1.f; return hipSuccess; } // no clock here: timings of a host run mean nothing
static inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }

// ---- device-side helpers ---------------------------------------------------------------------------
template <class A, class B, class = std::enable_if_t<std::is_arithmetic_v<A> && std::is_arithmetic_v<B>>>
static inline std::common_type_t<A, B> min(A a, B b) { using T = std::common_type_t<A, B>; return (T)a < (T)b ? (T)a : (T)b; }
template <class A, class B, class = std::enable_if_t<std::is_arithmetic_v<A> && std::is_arithmetic_v<B>>>
static inline std::common_type_t<A, B> max(A a, B b) { using T = std::common_type_t<A, B>; return (T)a > (T)b ? (T)a : (T)b; }

template <class T> static inline T atomicAdd(T* p, T v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
template <class T> static inline T atomicMax(T* p, T v) { T o = __atomic_load_n(p, __ATOMIC_SEQ_CST); while (o < v && !__atomic_compare_exchange_n(p, &o, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {} return o; }
template <class T> static inline T atomicExch(T* p, T v) { return __atomic_exchange_n(p, v, __ATOMIC_SEQ_CST); }
static inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }
static inline void __syncthreads() { emu::block_barrier(); }
static inline unsigned __lane_id() { return threadIdx.x & 63u; }

static inline int emu_src_lane_dpp(int lane, int ctrl, bool& valid)
{
    valid = true;
    const int row = lane & ~15, in = lane & 15;
    if (ctrl >= 0 && ctrl <= 0xFF) return (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);  // quad_perm
    if (ctrl >= 0x101 && ctrl <= 0x10F) { const int s = in + (ctrl & 15); valid = s < 16; return row | (s & 15); } // row_shl
    if (ctrl >= 0x111 && ctrl <= 0x11F) { const int s = in - (ctrl & 15); valid = s >= 0; return row | (s & 15); } // row_shr
    if (ctrl >= 0x121 && ctrl <= 0x12F) return row | ((in - (ctrl & 15)) & 15);                                    // row_ror
    if (ctrl == 0x140) return row | (15 - in);                                                                      // row_mirror
    if (ctrl == 0x141) return (lane & ~7) | (7 - (lane & 7));                                                      // row_half_mirror
    fprintf(stderr, "emu: DPP control 0x%x not modelled\n", ctrl);
    abort();
}
static inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl)
{
    const int lane = (int)(threadIdx.x & 63u);
    const uint64_t* all = emu::exchange((uint32_t)src);
    bool valid;
    const int from = emu_src_lane_dpp(lane, ctrl, valid);
    int r = valid ? (int)(uint32_t)all[from] : (bound_ctrl ? 0 : old);
    if (!((row_mask >> (lane >> 4)) & 1) || !((bank_mask >> ((lane >> 2) & 3)) & 1)) r = old;
    emu::exchange_done();
    return r;
}
static inline int emu_readlane(int v, int lane)
{
    const uint64_t* all = emu::exchange((uint32_t)v);
    const int r = (int)(uint32_t)all[lane & 63];
    emu::exchange_done();
    return r;
}
static inline int emu_bpermute(int addr, int v)
{
    const uint64_t* all = emu::exchange((uint32_t)v);
    const int r = (int)(uint32_t)all[(addr >> 2) & 63];
    emu::exchange_done();
    return r;
}
static inline uint64_t emu_ballot(bool p)
{
    const uint64_t* all = emu::exchange(p ? 1u : 0u);
    uint64_t m = 0;
    for (int i = 0; i < 64; i++) m |= (uint64_t)(all[i] & 1u) << i;
    emu::exchange_done();
    return m;
}
template <class T>
static inline T __shfl_up(T v, unsigned d)
{
    static_assert(sizeof(T) <= 8, "shuffle of at most 8 bytes");
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const uint64_t* all = emu::exchange(bits);
    const unsigned lane = threadIdx.x & 63u;
    T r = v;
    if (lane >= d) memcpy(&r, &all[lane - d], sizeof(T));
    emu::exchange_done();
    return r;
}
template <class T>
static inline T __shfl_xor(T v, int mask)
{
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const uint64_t* all = emu::exchange(bits);
    T r;
    memcpy(&r, &all[(threadIdx.x ^ mask) & 63u], sizeof(T));
    emu::exchange_done();
    return r;
}
template <class T>
static inline T __shfl(T v, int lane)
{
    uint64_t bits = 0;
    memcpy(&bits, &v, sizeof(T));
    const uint64_t* all = emu::exchange(bits);
    T r;
    memcpy(&r, &all[lane & 63], sizeof(T));
    emu::exchange_done();
    return r;
}

typedef _Float16 emu_half2 __attribute__((ext_vector_type(2)));
static inline float emu_fdot2(emu_half2 a, emu_half2 b, float c, bool)
{
    return ((float)a.x * (float)b.x + (float)a.y * (float)b.y) + c;
}
// v_cvt_pkrtz_f16_f32: two floats to halves, rounded toward zero
static inline _Float16 emu_rtz_half(float f)
{
    _Float16 h = (_Float16)f; // to nearest
    if (fabsf((float)h) > fabsf(f)) { // one step toward zero
        uint16_t b;
        memcpy(&b, &h, 2);
        b -= 1;
        memcpy(&h, &b, 2);
    }
    return h;
}
static inline emu_half2 emu_cvt_pkrtz(float a, float b) { return emu_half2{emu_rtz_half(a), emu_rtz_half(b)}; }
static inline uint32_t emu_alignbyte(uint32_t hi, uint32_t lo, uint32_t sh)
{
    return (uint32_t)((((uint64_t)hi << 32) | lo) >> (8 * (sh & 3u)));
}

// v_perm_b32: byte i of the result is byte sel[i] of {s0 : s1} (0..3 from s1, 4..7 from s0), 0x0c gives 0x00,
// 0x0d and above 0xff; the sign-replicating selectors 8..11 are modelled too.
static inline uint32_t emu_perm(uint32_t s0, uint32_t s1, uint32_t sel)
{
    const uint64_t src = ((uint64_t)s0 << 32) | s1;
    uint32_t r = 0;
    for (int i = 0; i < 4; i++) {
        const uint32_t c = (sel >> (8 * i)) & 0xFFu;
        uint32_t b;
        if (c <= 7) b = (uint32_t)(src >> (8 * c)) & 0xFFu;
        else if (c <= 11) b = ((src >> (16 * (c - 8) + 15)) & 1u) ? 0xFFu : 0u;
        else if (c == 12) b = 0;
        else b = 0xFFu;
        r |= b << (8 * i);
    }
    return r;
}

// v_mfma_f32_16x16x32_f16: lane l holds A[l % 16][8 * (l / 16) .. + 8), B[8 * (l / 16) .. + 8)[l % 16],
// and D[4 * (l / 16) + i][l % 16], i < 4.
typedef _Float16 emu_half8 __attribute__((ext_vector_type(8)));
typedef float emu_float4 __attribute__((ext_vector_type(4)));
emu_float4 emu_mfma_16x16x32_f16(emu_half8 a, emu_half8 b, emu_float4 c);

#define __builtin_amdgcn_update_dpp emu_update_dpp
#define __builtin_amdgcn_readlane emu_readlane
#define __builtin_amdgcn_ds_bpermute emu_bpermute
#define __builtin_amdgcn_ballot_w64 emu_ballot
#define __builtin_amdgcn_fdot2 emu_fdot2
#define __builtin_amdgcn_alignbyte emu_alignbyte
#define __builtin_amdgcn_perm emu_perm
#define __builtin_amdgcn_cvt_pkrtz emu_cvt_pkrtz
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) emu_mfma_16x16x32_f16(a, b, c)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
#define __builtin_amdgcn_wave_barrier() emu::wave_barrier()
#define __builtin_amdgcn_s_barrier() emu::block_barrier()
#define __builtin_nontemporal_load(p) (*(p))

#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_WORKGROUP 0
#define __HIP_MEMORY_SCOPE_SYSTEM 0
#define __hip_atomic_store(p, v, order, scope) \
    do { auto emu_v_ = (v); __atomic_store((p), &emu_v_, __ATOMIC_SEQ_CST); } while (0)
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)
#define __hip_atomic_load(p, order, scope) __atomic_load_n((p), __ATOMIC_SEQ_CST)
