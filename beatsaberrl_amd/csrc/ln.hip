// LayerNorm forward and residual-add + LayerNorm forward for gfx950.
//
// A row is owned by a group of LPR lanes of one wave64 (LPR = 16/32/64, so a
// wave carries 4/2/1 rows); each lane keeps NCH 16-byte chunks of the row in
// registers, the statistics are two butterfly reductions over the lane group
// (mean, then the centred sum of squares), all arithmetic in fp32.  The kernel
// is a pure HBM stream: 1 read + 1 write per element (2 + 2 for the add form).
//
// Semantics follow the reference's kernels (python/beat_arena_env/csrc/
// layer_norm.cu:58-134 fp32, :147-282 fp16 I/O): fp32 weight/bias/statistics,
// the add form writes x = round(a + (b + b_bias)) and normalises the ROUNDED x.
#include "ln_io.h"

namespace {

template <typename IO, int LPR, int NCH, bool ADD>
__global__ __launch_bounds__(256) void ln_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                 const float* __restrict__ bb, const float* __restrict__ w,
                                                 const float* __restrict__ bias, void* __restrict__ xo,
                                                 void* __restrict__ y, float* __restrict__ mean_o,
                                                 float* __restrict__ rstd_o, int64_t rows, int d, float eps) {
    typedef LnIO<IO> io;
    constexpr int VEC = io::VEC;
    constexpr int RPW = WAVE / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, rsub = lane / LPR;
    const int64_t row = ((int64_t)blockIdx.x * 4 + wave) * RPW + rsub;
    const bool rv = row < rows;
    const int64_t base = row * (int64_t)d;
    float v[NCH][VEC];
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int e0 = (c * LPR + sub) * VEC;
        const bool on = rv && e0 < d;
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[c][j] = 0.f;
        if (on) {
            io::load(a, base + e0, v[c]);
            if (ADD) {
                float t[VEC];
                io::load(b, base + e0, t);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float tb = bb ? t[j] + bb[e0 + j] : t[j];
                    v[c][j] = io::round(v[c][j] + tb);
                }
                io::store(xo, base + e0, v[c]);
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) s += v[c][j];
    }
    const float inv_d = 1.0f / (float)d;
    const float mean = group_sum<LPR>(s) * inv_d;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int e0 = (c * LPR + sub) * VEC;
        if (e0 < d) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) { float t = v[c][j] - mean; q += t * t; }
        }
    }
    const float var = group_sum<LPR>(q) * inv_d;
    const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int e0 = (c * LPR + sub) * VEC;
        if (rv && e0 < d) {
            float o[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = (v[c][j] - mean) * rstd * w[e0 + j] + bias[e0 + j];
            io::store(y, base + e0, o);
        }
    }
    if (rv && sub == 0) {
        if (mean_o) mean_o[row] = mean;
        if (rstd_o) rstd_o[row] = rstd;
    }
}

template <typename IO, int LPR, int NCH>
void launch(bool add, const void* a, const void* b, const float* bb, const float* w, const float* bias,
            void* x, void* y, float* mean, float* rstd, int64_t rows, int d, float eps, hipStream_t st) {
    constexpr int RPB = 4 * (WAVE / LPR);
    const unsigned grid = (unsigned)((rows + RPB - 1) / RPB);
    if (add) hipLaunchKernelGGL((ln_kernel<IO, LPR, NCH, true>), dim3(grid), dim3(256), 0, st, a, b, bb, w, bias, x, y, mean, rstd, rows, d, eps);
    else hipLaunchKernelGGL((ln_kernel<IO, LPR, NCH, false>), dim3(grid), dim3(256), 0, st, a, b, bb, w, bias, x, y, mean, rstd, rows, d, eps);
}

template <typename IO>
int dispatch(bool add, const void* a, const void* b, const float* bb, const float* w, const float* bias,
             void* x, void* y, float* mean, float* rstd, int64_t rows, int64_t d, float eps, hipStream_t st) {
    constexpr int VEC = LnIO<IO>::VEC;
    const int c16 = 16 * VEC, c32 = 32 * VEC, c64 = 64 * VEC;
#define LN_GO(LPR, NCH) do { launch<IO, LPR, NCH>(add, a, b, bb, w, bias, x, y, mean, rstd, rows, (int)d, eps, st); return BSRL_OK; } while (0)
    if (d <= c16) LN_GO(16, 1);
    if (d <= 2 * c16 && d % c16 == 0) LN_GO(16, 2);
    if (d <= c32) LN_GO(32, 1);
    if (d <= 3 * c16) LN_GO(16, 3);
    if (d <= 2 * c32) LN_GO(32, 2);
    if (d <= 3 * c32) LN_GO(32, 3);
    if (d <= 4 * c32) LN_GO(32, 4);
    if (d <= 4 * c64) LN_GO(64, 4);
    if (d <= 8 * c64) LN_GO(64, 8);
#undef LN_GO
    return BSRL_UNSUPPORTED;
}

int ln_entry(bool add, const void* a, const void* b, const float* bb, const float* w, const float* bias,
             void* x, void* y, float* mean, float* rstd, int64_t rows, int64_t d, float eps, int dtype,
             bsrl_stream stream) {
    const char* what = add ? "bsrl_ln_fwd_add" : "bsrl_ln_fwd";
    if (!a || !w || !bias || !y || (add && (!b || !x))) BSRL_FAIL(BSRL_EINVAL, "%s: null pointer", what);
    if (rows < 0 || d <= 0) BSRL_FAIL(BSRL_EINVAL, "%s: bad shape rows=%lld d=%lld", what, (long long)rows, (long long)d);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "%s: bad dtype %d", what, dtype);
    if (rows == 0) return BSRL_OK;
    const int vec = dtype == BSRL_F32 ? 4 : 8;
    if (d % vec != 0) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(a, 16) || !bsrl_aligned(y, 16) || (add && (!bsrl_aligned(b, 16) || !bsrl_aligned(x, 16))))
        return BSRL_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc;
    if (dtype == BSRL_F32) rc = dispatch<F32IO>(add, a, b, bb, w, bias, x, y, mean, rstd, rows, d, eps, st);
    else if (dtype == BSRL_F16) rc = dispatch<F16>(add, a, b, bb, w, bias, x, y, mean, rstd, rows, d, eps, st);
    else rc = dispatch<BF16>(add, a, b, bb, w, bias, x, y, mean, rstd, rows, d, eps, st);
    if (rc == BSRL_OK) BSRL_CHECK_LAUNCH(what);
    return rc;
}

}  // namespace

extern "C" int bsrl_ln_fwd(const void* x, const float* weight, const float* bias, void* y, float* mean,
                           float* rstd, int64_t rows, int64_t d, float eps, int dtype, bsrl_stream stream) {
    return ln_entry(false, x, nullptr, nullptr, weight, bias, nullptr, y, mean, rstd, rows, d, eps, dtype, stream);
}

extern "C" int bsrl_ln_fwd_add(const void* a, const void* b, const float* b_bias, const float* weight,
                               const float* bias, void* x, void* y, float* mean, float* rstd, int64_t rows,
                               int64_t d, float eps, int dtype, bsrl_stream stream) {
    return ln_entry(true, a, b, b_bias, weight, bias, x, y, mean, rstd, rows, d, eps, dtype, stream);
}
