// ref_wrap.cpp -- C entry points around the reference's own dequantisation header.
//
// TEST INFRASTRUCTURE ONLY.  This file contains no reference code: it includes
// src/quants.h from the mounted reference tree at build time (-I/root/reference/src,
// see the Makefile) and exposes its inline functions with C linkage so the tests can
// compare the oracle's restatement with the reference bit for bit.  The built library
// goes to oracle/_ref/ and is not committed.
#include <cstddef>
#include <cstdint>

#include "quants.h"

extern "C" {

float qkref_f16_to_f32(uint16_t h) { return qk_f16_to_f32(h); }
uint16_t qkref_f32_to_f16(float f) { return qk_f32_to_f16(f); }

size_t qkref_block_bytes(int type)
{
    switch (type) {
    case 8: return sizeof(block_q8_0);
    case 14: return sizeof(block_q6_K);
    case 23: return sizeof(block_iq4_xs);
    case 18: return sizeof(block_iq3_xxs);
    default: return 0;
    }
}

// type ids are ggml's: 8 Q8_0, 14 Q6_K, 18 IQ3_XXS, 23 IQ4_XS
int qkref_dequant_row(int type, const void* row, float* y, int64_t k)
{
    switch (type) {
    case 8: dequant_row_q8_0((const block_q8_0*)row, y, k); return 0;
    case 14: dequant_row_q6_K((const block_q6_K*)row, y, k); return 0;
    case 23: dequant_row_iq4_xs((const block_iq4_xs*)row, y, k); return 0;
    case 18: dequant_row_iq3_xxs((const block_iq3_xxs*)row, y, k); return 0;
    default: return -1;
    }
}

uint32_t qkref_iq3xxs_grid(uint32_t i) { return iq3xxs_grid[i & 255u]; }
uint8_t qkref_ksigns(uint32_t i) { return ksigns_iq2xs[i & 127u]; }
uint8_t qkref_kmask(uint32_t i) { return kmask_iq2xs[i & 7u]; }
int8_t qkref_iq4nl(uint32_t i) { return kvalues_iq4nl[i & 15u]; }

// Row dot in double over a dequantised row: the loop every caseXXX builder runs
// (the statement itself is ours; only dequant_row_* comes from the reference).
int qkref_gemv(int type, const void* W, size_t row_bytes, const float* x, float* y, uint32_t M,
               uint32_t K, float* scratch)
{
    for (uint32_t m = 0; m < M; m++) {
        if (qkref_dequant_row(type, (const uint8_t*)W + (size_t)m * row_bytes, scratch, K)) return -1;
        double acc = 0;
        for (uint32_t k = 0; k < K; k++) acc += (double)scratch[k] * x[k];
        y[m] = (float)acc;
    }
    return 0;
}
}
