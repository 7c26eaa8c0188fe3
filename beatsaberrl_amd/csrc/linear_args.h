// Argument block shared by the linear kernels.
#pragma once
#include "bsrl_common.h"

struct LinArgs {
    const void* x; int64_t ldx;
    const void* w;
    const float* bias;
    const void* res; int64_t ldr;
    void* y; int64_t ldy;
    void* y2; int64_t ldy2; int64_t split;
    int64_t rows; int K; int M;
    int out_f32;
};

// LDS-tiled 16-bit kernel for large row counts (linear_tiled.hip); returns false when the
// shape is outside what it covers (the caller then takes the direct-from-global kernel).
bool bsrl_linear_tiled(const LinArgs& a, int act, int dtype, hipStream_t st);
