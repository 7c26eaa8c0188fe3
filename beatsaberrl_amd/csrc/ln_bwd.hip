// LayerNorm backward for gfx950: dx per row, dw / db (/ dbb) as column sums over all rows.
//
// Replaces the reference's ln_bwd (python/beat_arena_env/csrc/layer_norm.cu:284-420 kernels,
// :645-729 host side) behind _LnFn / _LnAddFn.backward (python/fused_ln.py:56-112):
//     xhat = (x - mean) * rstd,  g = dy * w,  s1 = sum(g) / d,  s2 = sum(g * xhat) / d
//     dx   = (g - s1 - xhat * s2) * rstd  (+ gx, the residual-path gradient, before the one rounding)
//     dw   = sum_rows dy * xhat,  db = sum_rows dy,  dbb = sum_rows of the STORED (rounded) dx
// all in fp32 on fp32 / fp16 / bf16 activations.
//
// Same lane layout as the forward: a row is owned by LPR lanes that keep NCH 16-byte chunks in
// registers.  A workgroup walks rows with a grid stride and every lane accumulates its columns'
// dw / db / dbb in registers; at the end the 4 waves' row slots are summed in a fixed order through
// LDS into one partial row per workgroup, and a second kernel sums the partials per column, again
// in a fixed order: the result is reproducible run to run (no float atomics), which is what the
// reference's fixed-size partials + torch.sum achieve (layer_norm.cu:668-676).
// HBM traffic: x, dy (and gx) read once, dx written once; the partials are <= 2048 rows of d.
#include "ln_io.h"

namespace {

constexpr int LNB_MAX_GRID = 2048;

template <typename IO, int LPR, int NCH, bool DBB>
__global__ __launch_bounds__(256) void ln_bwd_kernel(const void* __restrict__ x, const void* __restrict__ dy,
                                                     const float* __restrict__ w, const float* __restrict__ mean,
                                                     const float* __restrict__ rstd, const void* __restrict__ gx,
                                                     void* __restrict__ dx, float* __restrict__ part,
                                                     int64_t rows, int d) {
    typedef LnIO<IO> io;
    constexpr int VEC = io::VEC;
    constexpr int RPW = WAVE / LPR, SLOTS = 4 * RPW, DCAP = LPR * NCH * VEC;
    __shared__ float sm[SLOTS * DCAP];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, rsub = lane / LPR;
    const float inv_d = 1.0f / (float)d;
    float wv[NCH][VEC], aw[NCH][VEC], ab[NCH][VEC], abb[DBB ? NCH : 1][VEC];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int e0 = (c * LPR + sub) * VEC;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            wv[c][j] = e0 < d ? w[e0 + j] : 0.f;
            aw[c][j] = 0.f; ab[c][j] = 0.f;
            if (DBB) abb[c][j] = 0.f;
        }
    }
    // the next pass's x / dy are in flight (raw registers) while this pass computes
    typename io::raw nx[NCH], ng[NCH];
    float nmu = 0.f, nr = 0.f;
    auto fetch = [&](int64_t rb) {
        const int64_t row = (rb * 4 + wave) * RPW + rsub;
        nmu = row < rows ? mean[row] : 0.f;
        nr = row < rows ? rstd[row] : 0.f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int e0 = (c * LPR + sub) * VEC;
            if (row < rows && e0 < d) { nx[c] = io::load_raw(x, row * (int64_t)d + e0); ng[c] = io::load_raw(dy, row * (int64_t)d + e0); }
        }
    };
    if ((int64_t)blockIdx.x * SLOTS < rows) fetch(blockIdx.x);
    for (int64_t rb = blockIdx.x; rb * SLOTS < rows; rb += gridDim.x) {
        const int64_t row = (rb * 4 + wave) * RPW + rsub;
        const bool rv = row < rows;
        const int64_t base = row * (int64_t)d;
        const float mu = nmu, r = nr;
        float xh[NCH][VEC], g[NCH][VEC];
        float s1 = 0.f, s2 = 0.f;
        typename io::raw cx[NCH], cg[NCH];
#pragma unroll
        for (int c = 0; c < NCH; ++c) { cx[c] = nx[c]; cg[c] = ng[c]; }
        if ((rb + gridDim.x) * SLOTS < rows) fetch(rb + gridDim.x);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int e0 = (c * LPR + sub) * VEC;
            float xv[VEC], gv[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) { xv[j] = 0.f; gv[j] = 0.f; }
            if (rv && e0 < d) { io::cvt(cx[c], xv); io::cvt(cg[c], gv); }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                xh[c][j] = (xv[j] - mu) * r;                 // 0 for rows past the end (r = 0, x = mu = 0)
                g[c][j] = gv[j] * wv[c][j];
                s1 += g[c][j];
                s2 += g[c][j] * xh[c][j];
                aw[c][j] += gv[j] * xh[c][j];
                ab[c][j] += gv[j];
            }
        }
        s1 = group_sum<LPR>(s1) * inv_d;
        s2 = group_sum<LPR>(s2) * inv_d;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int e0 = (c * LPR + sub) * VEC;
            if (rv && e0 < d) {
                float o[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) o[j] = (g[c][j] - s1 - xh[c][j] * s2) * r;
                if (gx) {
                    float t[VEC];
                    io::load(gx, base + e0, t);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o[j] += t[j];
                }
                io::store(dx, base + e0, o);
                if (DBB) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) abb[c][j] += io::round(o[j]);
                }
            }
        }
    }
    // fold the workgroup's row slots, one quantity at a time, in slot order
    float* out = part + (int64_t)blockIdx.x * (DBB ? 3 : 2) * d;
#pragma unroll
    for (int q = 0; q < (DBB ? 3 : 2); ++q) {
        if (q) __syncthreads();
#pragma unroll
        for (int c = 0; c < NCH; ++c)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                sm[(wave * RPW + rsub) * DCAP + (c * LPR + sub) * VEC + j] = q == 0 ? aw[c][j] : q == 1 ? ab[c][j] : abb[DBB ? c : 0][j];
        __syncthreads();
        for (int col = threadIdx.x; col < d; col += 256) {
            float t = 0.f;
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) t += sm[s * DCAP + col];
            out[q * d + col] = t;
        }
    }
}

// dw / db / dbb[col] = sum over the G partial rows: a workgroup owns 16 columns, its 16 row slices run interleaved
// sums that are folded in slice order (a fixed order: reproducible)
__global__ __launch_bounds__(256) void ln_bwd_reduce_kernel(const float* __restrict__ part, int G, int nq, int d,
                                                            float* __restrict__ dw, float* __restrict__ db,
                                                            float* __restrict__ dbb) {
    __shared__ float sm[16][17];
    const int cl = threadIdx.x & 15, k = threadIdx.x >> 4;
    const int q = blockIdx.y, col = blockIdx.x * 16 + cl;
    float t = 0.f;
    if (col < d)
        for (int gi = k; gi < G; gi += 16) t += part[((int64_t)gi * nq + q) * d + col];
    sm[k][cl] = t;
    __syncthreads();
    if (k == 0 && col < d) {
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) v += sm[j][cl];
        (q == 0 ? dw : q == 1 ? db : dbb)[col] = v;
    }
}

// workgroups that are resident at once on the current device: the persistent grid is one such round, so that no
// workgroup waits for a slot while others are already in their tail
template <typename K> int resident_grid(K kernel) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || cus < 1 || per_cu < 1)
        return LNB_MAX_GRID;
    const int64_t g = (int64_t)cus * per_cu;
    return g < LNB_MAX_GRID ? (int)g : LNB_MAX_GRID;
}

template <typename IO, int LPR, int NCH>
void launch(const void* x, const void* dy, const float* w, const float* mean, const float* rstd, const void* gx,
            void* dx, float* part, bool dbb, int64_t rows, int d, int* grid_io, hipStream_t st) {
    // one cap for both forms, so that dw / db do not depend on whether dbb was asked for
    static const int cap = [] { const int c0 = resident_grid(ln_bwd_kernel<IO, LPR, NCH, false>), c1 = resident_grid(ln_bwd_kernel<IO, LPR, NCH, true>);
                                return c0 < c1 ? c0 : c1; }();
    const int grid = *grid_io < cap ? *grid_io : cap;
    *grid_io = grid;
    if (dbb) hipLaunchKernelGGL((ln_bwd_kernel<IO, LPR, NCH, true>), dim3(grid), dim3(256), 0, st, x, dy, w, mean, rstd, gx, dx, part, rows, d);
    else hipLaunchKernelGGL((ln_bwd_kernel<IO, LPR, NCH, false>), dim3(grid), dim3(256), 0, st, x, dy, w, mean, rstd, gx, dx, part, rows, d);
}

// rows per workgroup pass (4 waves x 64 / LPR) for the lane layout picked for d, 0 = no kernel
template <typename IO> int pick(int64_t d, int* lpr, int* nch) {
    constexpr int VEC = LnIO<IO>::VEC;
    const int c16 = 16 * VEC, c32 = 32 * VEC, c64 = 64 * VEC;
    if (d <= c16) { *lpr = 16; *nch = 1; }
    else if (d <= 2 * c16 && d % c16 == 0) { *lpr = 16; *nch = 2; }
    else if (d <= c32) { *lpr = 32; *nch = 1; }
    else if (d <= 3 * c16) { *lpr = 16; *nch = 3; }
    else if (d <= 2 * c32) { *lpr = 32; *nch = 2; }
    else if (d <= 3 * c32) { *lpr = 32; *nch = 3; }
    else if (d <= 4 * c32) { *lpr = 32; *nch = 4; }
    else if (d <= 4 * c64) { *lpr = 64; *nch = 4; }
    else return 0;
    return 4 * (WAVE / *lpr);
}

template <typename IO>
int dispatch(const void* x, const void* dy, const float* w, const float* mean, const float* rstd, const void* gx,
             void* dx, float* part, bool dbb, int64_t rows, int64_t d, int* grid_out, hipStream_t st) {
    int lpr, nch;
    const int rpb = pick<IO>(d, &lpr, &nch);
    if (!rpb) return BSRL_UNSUPPORTED;
    const int64_t want = (rows + rpb - 1) / rpb;
    *grid_out = (int)(want < LNB_MAX_GRID ? want : LNB_MAX_GRID);
#define LNB_GO(LPR, NCH) if (lpr == LPR && nch == NCH) { launch<IO, LPR, NCH>(x, dy, w, mean, rstd, gx, dx, part, dbb, rows, (int)d, grid_out, st); return BSRL_OK; }
    LNB_GO(16, 1) LNB_GO(16, 2) LNB_GO(32, 1) LNB_GO(16, 3) LNB_GO(32, 2) LNB_GO(32, 3) LNB_GO(32, 4) LNB_GO(64, 4)
#undef LNB_GO
    return BSRL_UNSUPPORTED;
}

}  // namespace

extern "C" int64_t bsrl_ln_bwd_workspace_size(int64_t d) {
    return d > 0 ? (int64_t)LNB_MAX_GRID * 3 * d * (int64_t)sizeof(float) : 0;
}

extern "C" int bsrl_ln_bwd(const void* x, const void* dy, const float* weight, const float* mean, const float* rstd,
                           const void* gx, void* dx, float* dw, float* db, float* dbb, void* workspace,
                           int64_t rows, int64_t d, int dtype, bsrl_stream stream) {
    if (!weight || !dw || !db || !workspace || (rows > 0 && (!x || !dy || !mean || !rstd || !dx)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_bwd: null pointer");
    if (rows < 0 || d <= 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_bwd: bad shape rows=%lld d=%lld", (long long)rows, (long long)d);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_bwd: bad dtype %d", dtype);
    const int vec = dtype == BSRL_F32 ? 4 : 8;
    if (d % vec != 0) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(x, 16) || !bsrl_aligned(dy, 16) || !bsrl_aligned(dx, 16) || (gx && !bsrl_aligned(gx, 16)))
        return BSRL_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    float* part = static_cast<float*>(workspace);
    const int nq = dbb ? 3 : 2;
    int grid = 0, rc;
    if (rows == 0) rc = BSRL_OK;             // the reduce below then writes zeros (G = 0)
    else if (dtype == BSRL_F32) rc = dispatch<F32IO>(x, dy, weight, mean, rstd, gx, dx, part, dbb != nullptr, rows, d, &grid, st);
    else if (dtype == BSRL_F16) rc = dispatch<F16>(x, dy, weight, mean, rstd, gx, dx, part, dbb != nullptr, rows, d, &grid, st);
    else rc = dispatch<BF16>(x, dy, weight, mean, rstd, gx, dx, part, dbb != nullptr, rows, d, &grid, st);
    if (rc != BSRL_OK) return rc;
    hipLaunchKernelGGL(ln_bwd_reduce_kernel, dim3((unsigned)((d + 15) / 16), nq), dim3(256), 0, st, part, grid, nq, (int)d, dw, db, dbb);
    BSRL_CHECK_LAUNCH("bsrl_ln_bwd");
    return BSRL_OK;
}
