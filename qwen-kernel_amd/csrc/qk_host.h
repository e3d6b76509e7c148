// qk_host.h -- host-side plumbing shared by the launchers: error slot, argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/qk_kernels.h"

namespace qk {

// Records the message returned by qkk_last_error() and hands back `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Device probe shared by every launcher: QKK_OK when a HIP device is current.
int require_device();

// Blocks of 256 threads that fill the device four deep (16 waves per CU): the grid size of
// the streaming kernels, which loop over their work with a grid stride.
uint32_t persistent_blocks();

// Converts the last launch error (if any) into a QKK_EDEVICE failure.
int check_launch(const char* what);

// Switches of the library, read once from the environment on first use; qkk_set_option changes one at
// run time (a test or a bench that runs both forms of a kernel in one process).  A form of a kernel
// that has not yet been run and timed on a device is reached only through its switch: the default
// of every switch is the form that has.
struct Options {
    int one_row_stream = 0; // QK_ONE_ROW=stream: one-row GEMV / MoE step / LM head stream block rows as 16-byte pieces through LDS (default "lane": every lane loads its own block fields)
    int dense_reg = 0;      // QK_DENSE_REG=1: F16 / F32 GEMV keeps its share of x in registers
    int fused_norm = 0;     // QK_FUSED_NORM=1: the engine's one-row step folds each RMS norm into its consumer (needs the streaming form)
    int attn_block = 0;     // QK_ATTN_BLOCK=1: prefill attention over blocks of 16 rows on the matrix cores (default: two rows per workgroup)
    int dn_fused = 0;       // QK_DN_FUSED=1: the gated-DeltaNet decode step as one launch
    int gemm_tiled = 0;     // QK_GEMM_TILED=1: 64 and more activation rows go through the kernel that decodes every weight tile once per 128 rows
    int select_ranked = 1;  // QK_SELECT_RANKED=0: the streamed gate/up launch selects with wave 0's rounds (as the per-lane form does) instead of by rank counting on all four waves
    int head_rows = 0;      // QK_HEAD_ROWS=1: the LM head for 2..16 rows with the waves splitting the vocabulary rows instead of K
    int moe_rows = 0;       // QK_MOE_ROWS=1: the routed experts' projections for more than ten rows with the waves splitting the weight rows instead of K
    int gemv_depth = 0;     // QK_GEMV_DEPTH=n (1..16): workgroups per CU of the streaming GEMV's persistent grid, 0 = built-in
    int head_depth = 0;     // QK_HEAD_DEPTH=n (1..8): the same for the streaming LM head
    int rowwise_max = 0;    // QK_ROWWISE_MAX=n (1..64): rows up to which the plain MoE step runs row by row, 0 = QKK_ROWWISE_MAX
};
Options& options();
void apply_env_options(Options& v); // qk_open reads the environment again: switches set since the first use take effect for the engine it builds

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

} // namespace qk
