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

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

} // namespace qk
