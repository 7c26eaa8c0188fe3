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
    // grouped output rows (0 = off): output row r lives at (r / y_group) * y_gstride + (r % y_group) * ldy,
    // i.e. y is a (rows / y_group, y_group, M) view of a larger tensor (a token slice of a (B, T, d) stream)
    int y_group; int64_t y_gstride;
    // ReLU gate (NULL = off): the result is kept where gate[row * ldgate + col] > 0 and zeroed elsewhere - the
    // backward of a ReLU whose forward output is `gate`, applied in the epilogue of the data-gradient GEMM
    const void* gate; int64_t ldgate;
};

// element offset of output row `row` in y (rows < 2^31 is checked on the host)
__device__ __forceinline__ int64_t lin_yoff(const LinArgs& a, int64_t row) {
    if (a.y_group == 0) return row * a.ldy;
    const uint32_t r = (uint32_t)row, gq = r / (uint32_t)a.y_group;
    return (int64_t)gq * a.y_gstride + (int64_t)(r - gq * (uint32_t)a.y_group) * a.ldy;
}

// LDS-tiled 16-bit kernel for large row counts (linear_tiled.hip); returns false when the
// shape is outside what it covers (the caller then takes the direct-from-global kernel).
bool bsrl_linear_tiled(const LinArgs& a, int act, int dtype, hipStream_t st);

// Weight-resident streaming 16-bit kernel for many rows and K = 128 / 192 / 256 / 384 (linear_stream.hip);
// false when the shape is outside what it covers.
bool bsrl_linear_stream(const LinArgs& a, int act, int dtype, hipStream_t st);

// Two Linears with a ReLU between them in one launch (linear_stream.hip): x (rows, K1) -> relu(x W1^T + b1) -> l2 (its
// w, bias, y, grouping; K = M = d); false when the shape is outside what it covers (K1 = 64, d = 128 / 192, 16-bit).
bool bsrl_mlp2_stream(const LinArgs& l2, const void* x, int64_t ldx, const void* w1, const float* b1, int64_t K1, int dtype,
                      hipStream_t st);

// Ring-buffered 16-bit kernel for large row counts and K a multiple of 32 (linear_ring.hip): operands go from
// global memory straight into an LDS ring; false when the shape is outside what it covers.
bool bsrl_linear_ring(const LinArgs& a, int act, int dtype, hipStream_t st);
