// Row-wise stages of two architecture options of the policy, and the ReLU gradient mask; HBM-bound
// elementwise / row-reduction work.
//
//  * ReLU backward (reference fp16_gemm.relu_bwd, python/beat_arena_env/csrc/fp16_gemm.cu:113-187): gm = g * [y > 0]
//    from the saved post-ReLU y, for a ReLU whose consumer is not a GEMM this library can gate.
//  * value-residual mix (reference python/fp16_linear.py:1002-1006, python/policy.py:568-611):
//        out = a * v + b * v0      fp32 arithmetic, rounded once to the stream dtype; (a, b) live on the device
//    (learned scalars), exactly v at (a, b) = (1, 0).
//  * SimBaV2 readout stages (reference python/policy.py:1140-1155, l2n :742-744): scalers, ReLU, row l2
//    normalisation x / max(|x|, 1e-6) and the LERP in fp32 between the trunk's three GEMMs, each stored value
//    rounded once.
//
// Rows are independent and a row's result never depends on the launch shape: one wave owns a row (fixed
// butterfly reduction order), one thread owns 8 (16-bit) or 4 (fp32) consecutive elements of the mix.
#include "bsrl_common.h"

namespace {

template <typename IO> struct El;
template <> struct El<F16> { typedef u16 T; static __device__ __forceinline__ float f(u16 v) { return F16::to_f(v); }
                             static __device__ __forceinline__ u16 r(float v) { return F16::from_f(v); } };
template <> struct El<BF16> { typedef u16 T; static __device__ __forceinline__ float f(u16 v) { return BF16::to_f(v); }
                              static __device__ __forceinline__ u16 r(float v) { return BF16::from_f(v); } };
template <> struct El<F32IO> { typedef float T; static __device__ __forceinline__ float f(float v) { return v; }
                               static __device__ __forceinline__ float r(float v) { return v; } };

struct MixArgs {
    const void* v; int64_t ldv; const void* v0; int64_t ldv0; const float* a; const float* b;
    void* out; int64_t ldo; int64_t rows; int d;
};

// VEC consecutive elements per thread; the host picks VEC > 1 only when every row start is VEC-element aligned
template <typename IO, int VEC>
__global__ __launch_bounds__(256) void vres_mix_kernel(MixArgs m) {
    typedef typename El<IO>::T T;
    const int per_row = m.d / VEC;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= m.rows * per_row) return;
    const int64_t row = i / per_row; const int c = (int)(i % per_row) * VEC;
    const float a = *m.a, b = *m.b;
    const T* pv = static_cast<const T*>(m.v) + row * m.ldv + c;
    const T* p0 = static_cast<const T*>(m.v0) + row * m.ldv0 + c;
    T* po = static_cast<T*>(m.out) + row * m.ldo + c;
    if (VEC > 1) {
        typedef T TV __attribute__((ext_vector_type(VEC > 1 ? VEC : 2)));
        const TV xv = *reinterpret_cast<const TV*>(pv), x0 = *reinterpret_cast<const TV*>(p0);
        TV o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const float t = El<IO>::f(xv[j]) * a;                   // v * a, rounded to fp32 ...
            o[j] = El<IO>::r(fmaf(El<IO>::f(x0[j]), b, t));         // ... then + v0 * b accumulated in fp32
        }
        *reinterpret_cast<TV*>(po) = o;
    } else {
        *po = El<IO>::r(fmaf(El<IO>::f(*p0), b, El<IO>::f(*pv) * a));
    }
}

// gradient through a ReLU: out = g where the ReLU's forward output y is positive, 0 elsewhere
template <typename IO, int VEC>
__global__ __launch_bounds__(256) void relu_bwd_kernel(MixArgs m) {
    typedef typename El<IO>::T T;
    const int per_row = m.d / VEC;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= m.rows * per_row) return;
    const int64_t row = i / per_row; const int c = (int)(i % per_row) * VEC;
    const T* pg = static_cast<const T*>(m.v) + row * m.ldv + c;
    const T* py = static_cast<const T*>(m.v0) + row * m.ldv0 + c;
    T* po = static_cast<T*>(m.out) + row * m.ldo + c;
    if (VEC > 1) {
        typedef T TV __attribute__((ext_vector_type(VEC > 1 ? VEC : 2)));
        const TV gv = *reinterpret_cast<const TV*>(pg), yv = *reinterpret_cast<const TV*>(py);
        TV o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = El<IO>::f(yv[j]) > 0.f ? gv[j] : (T)0;
        *reinterpret_cast<TV*>(po) = o;
    } else {
        *po = El<IO>::f(*py) > 0.f ? *pg : (T)0;
    }
}

struct HsArgs {
    int op; const void* t; const float* s; float c; const float* x32_in; float* x32_out; void* x_out;
    int64_t rows; int D;
};

__device__ __forceinline__ float inv_l2(float sumsq) { return 1.0f / fmaxf(sqrtf(sumsq), 1e-6f); }

// one wave per row; the row is re-read from cache for each pass instead of being held in registers
template <typename IO>
__global__ __launch_bounds__(256) void hsphere_kernel(HsArgs h) {
    typedef typename El<IO>::T T;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= h.rows) return;
    const int D = h.D;
    const T* t = static_cast<const T*>(h.t) + row * D;
    T* xo = h.x_out ? static_cast<T*>(h.x_out) + row * D : nullptr;
    if (h.op == BSRL_HS_SCALE_RELU) {
        for (int c = lane; c < D; c += 64) xo[c] = El<IO>::r(fmaxf(El<IO>::f(t[c]) * (h.s[c] * h.c), 0.0f));
        return;
    }
    if (h.op == BSRL_HS_SCALE_L2N) {
        float ss = 0.f;
        for (int c = lane; c < D; c += 64) { const float v = El<IO>::f(t[c]) * (h.s[c] * h.c); ss += v * v; }
        const float inv = inv_l2(group_sum<64>(ss));
        float* x32 = h.x32_out + row * D;
        for (int c = lane; c < D; c += 64) {
            const float v = El<IO>::f(t[c]) * (h.s[c] * h.c) * inv;
            x32[c] = v;
            if (xo) xo[c] = El<IO>::r(v);
        }
        return;
    }
    // BSRL_HS_L2N_LERP: y = l2n(t); z = x + alpha (y - x); out = sqrt(D) l2n(z)
    const float* x32 = h.x32_in + row * D;
    float ss = 0.f;
    for (int c = lane; c < D; c += 64) { const float v = El<IO>::f(t[c]); ss += v * v; }
    const float inv_y = inv_l2(group_sum<64>(ss));
    float zz = 0.f;
    for (int c = lane; c < D; c += 64) {
        const float x = x32[c], y = El<IO>::f(t[c]) * inv_y;
        const float z = x + (h.s[c] * h.c) * (y - x);
        zz += z * z;
    }
    const float inv_z = inv_l2(group_sum<64>(zz));
    const float root = sqrtf((float)D);
    for (int c = lane; c < D; c += 64) {
        const float x = x32[c], y = El<IO>::f(t[c]) * inv_y;
        const float z = x + (h.s[c] * h.c) * (y - x);
        xo[c] = El<IO>::r(z * inv_z * root);
    }
}

template <typename IO>
int mix_launch(const MixArgs& m, int vec, bool relu, hipStream_t st) {
    const int64_t n = m.rows * (m.d / vec);
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (relu) {
        if (vec == 8) hipLaunchKernelGGL((relu_bwd_kernel<IO, 8>), grid, block, 0, st, m);
        else if (vec == 4) hipLaunchKernelGGL((relu_bwd_kernel<IO, 4>), grid, block, 0, st, m);
        else hipLaunchKernelGGL((relu_bwd_kernel<IO, 1>), grid, block, 0, st, m);
    } else {
        if (vec == 8) hipLaunchKernelGGL((vres_mix_kernel<IO, 8>), grid, block, 0, st, m);
        else if (vec == 4) hipLaunchKernelGGL((vres_mix_kernel<IO, 4>), grid, block, 0, st, m);
        else hipLaunchKernelGGL((vres_mix_kernel<IO, 1>), grid, block, 0, st, m);
    }
    BSRL_CHECK_LAUNCH(relu ? "bsrl_relu_bwd" : "bsrl_vres_mix");
    return BSRL_OK;
}

// shared argument checks and dispatch of the two elementwise (rows, d) kernels above
int mix_entry(const char* what, bool relu, const void* v, int64_t ldv, const void* v0, int64_t ldv0, const float* a,
              const float* b, void* out, int64_t ldo, int64_t rows, int64_t d, int dtype, bsrl_stream stream) {
    if (!v || !v0 || !out || (!relu && (!a || !b))) BSRL_FAIL(BSRL_EINVAL, "%s: null pointer", what);
    if (rows < 0 || d < 1 || d > (1 << 20) || ldv < d || ldv0 < d || ldo < d)
        BSRL_FAIL(BSRL_EINVAL, "%s: need rows >= 0, 1 <= d <= 2^20 and row pitches >= d", what);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "%s: bad dtype %d", what, dtype);
    if (rows == 0) return BSRL_OK;
    if (rows * d > ((int64_t)1 << 40)) BSRL_FAIL(BSRL_EINVAL, "%s: rows * d too large", what);
    const int want = dtype == BSRL_F32 ? 4 : 8;                    // 16-byte accesses
    const bool vec_ok = d % want == 0 && ldv % want == 0 && ldv0 % want == 0 && ldo % want == 0 &&
                        bsrl_aligned(v, 16) && bsrl_aligned(v0, 16) && bsrl_aligned(out, 16);
    const int vec = vec_ok ? want : 1;
    if ((rows * (d / vec) + 255) / 256 > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "%s: grid too large", what);
    const MixArgs m{v, ldv, v0, ldv0, a, b, out, ldo, rows, (int)d};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == BSRL_F32) return mix_launch<F32IO>(m, vec, relu, st);
    if (dtype == BSRL_F16) return mix_launch<F16>(m, vec, relu, st);
    return mix_launch<BF16>(m, vec, relu, st);
}

// softmax(logits) . centers per row: one wave per row, the row's lanes strided over the bins (three passes over
// registers: max, sum of exponentials, weighted sum)
__global__ __launch_bounds__(256) void softmax_expect_kernel(const float* __restrict__ logits, const float* __restrict__ centers,
                                                             float* __restrict__ out, int64_t rows, int n) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* lr = logits + row * n;
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, lr[i]);
    m = group_max<64>(m);
    float se = 0.f, sc = 0.f;
    for (int i = lane; i < n; i += 64) {
        const float e = expf(lr[i] - m);
        se += e; sc = fmaf(e, centers[i], sc);
    }
    se = group_sum<64>(se); sc = group_sum<64>(sc);
    if (lane == 0) out[row] = sc / se;
}

}  // namespace

extern "C" int bsrl_softmax_expect(const float* logits, const float* centers, float* out, int64_t rows, int64_t n,
                                   bsrl_stream stream) {
    if (!logits || !centers || !out) BSRL_FAIL(BSRL_EINVAL, "bsrl_softmax_expect: null pointer");
    if (rows < 0 || n < 1 || n > 65536) BSRL_FAIL(BSRL_EINVAL, "bsrl_softmax_expect: need rows >= 0 and 1 <= n <= 65536");
    if (rows == 0) return BSRL_OK;
    if ((rows + 3) / 4 > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_softmax_expect: too many rows");
    hipLaunchKernelGGL(softmax_expect_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       logits, centers, out, rows, (int)n);
    BSRL_CHECK_LAUNCH("bsrl_softmax_expect");
    return BSRL_OK;
}

extern "C" int bsrl_vres_mix(const void* v, int64_t ldv, const void* v0, int64_t ldv0, const float* a, const float* b,
                             void* out, int64_t ldo, int64_t rows, int64_t d, int dtype, bsrl_stream stream) {
    return mix_entry("bsrl_vres_mix", false, v, ldv, v0, ldv0, a, b, out, ldo, rows, d, dtype, stream);
}

extern "C" int bsrl_relu_bwd(const void* g, int64_t ldg, const void* y, int64_t ldy, void* out, int64_t ldo,
                             int64_t rows, int64_t d, int dtype, bsrl_stream stream) {
    return mix_entry("bsrl_relu_bwd", true, g, ldg, y, ldy, nullptr, nullptr, out, ldo, rows, d, dtype, stream);
}

extern "C" int bsrl_hsphere(int op, const void* t, const float* s, float c, const float* x32_in, float* x32_out,
                            void* x_out, int64_t rows, int64_t D, int dtype, bsrl_stream stream) {
    if (op != BSRL_HS_SCALE_L2N && op != BSRL_HS_SCALE_RELU && op != BSRL_HS_L2N_LERP)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: unknown op %d", op);
    if (!t || !s) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: null input / scaler");
    if (op == BSRL_HS_SCALE_L2N && !x32_out) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: SCALE_L2N needs x32_out");
    if (op == BSRL_HS_SCALE_RELU && !x_out) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: SCALE_RELU needs x_out");
    if (op == BSRL_HS_L2N_LERP && (!x32_in || !x_out)) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: L2N_LERP needs x32_in and x_out");
    if (rows < 0 || D < 1 || D > 65536) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: need rows >= 0 and 1 <= D <= 65536");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: bad dtype %d", dtype);
    if (rows == 0) return BSRL_OK;
    if ((rows + 3) / 4 > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_hsphere: too many rows");
    const HsArgs h{op, t, s, c, x32_in, x32_out, x_out, rows, (int)D};
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == BSRL_F32) hipLaunchKernelGGL(hsphere_kernel<F32IO>, grid, block, 0, st, h);
    else if (dtype == BSRL_F16) hipLaunchKernelGGL(hsphere_kernel<F16>, grid, block, 0, st, h);
    else hipLaunchKernelGGL(hsphere_kernel<BF16>, grid, block, 0, st, h);
    BSRL_CHECK_LAUNCH("bsrl_hsphere");
    return BSRL_OK;
}
