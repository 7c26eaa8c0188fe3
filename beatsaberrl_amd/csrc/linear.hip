// y = act(x W^T + b) (+ residual) for gfx950.
//
// 16-bit path: v_mfma_f32_16x16x32 (f16 / bf16), fp32 accumulate.  A workgroup
// of 4 waves owns a 128-row x 128-column output tile (2 x 2 waves, each a
// 64 x 64 tile = 4 x 4 MFMA tiles, 64 accumulator VGPRs).  Both operands are
// read straight from global memory in MFMA fragment order: the weight is the
// MFMA "A" operand (its M index is the OUTPUT column), the activation the "B"
// operand (its N index is the ROW), so every lane ends up with 4 consecutive
// output columns of one row and the epilogue stores 8 or 16 bytes per lane.
// nn.Linear's (M, K) row-major weight is already K-contiguous per output
// column, which is exactly the fragment order.  All weights of this model are
// <= 1.2 MB and stay L2 resident; the kernel is an HBM stream over x and y.
//
// fp32 path: a plain LDS-tiled FMA kernel (parity configuration only).
//
// Replaces the vendor GEMM calls of the reference's op layer
// (python/fp16_linear.py:134-181) and the bias+ReLU epilogues of
// python/beat_arena_env/csrc/fp16_gemm.cu:77-111, 404-497.
#include "linear_args.h"

namespace {

// 8 consecutive k of one row, zero beyond K.  FAST: 16-byte aligned rows.
template <bool FAST>
__device__ __forceinline__ s16x8 load_frag(const u16* base, int64_t ld, int64_t row, int k0, int K) {
    s16x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
    const u16* p = base + row * ld + k0;
    if (FAST) {
        if (k0 < K) r = *reinterpret_cast<const s16x8*>(p);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) if (k0 + j < K) r[j] = (short)p[j];
    }
    return r;
}

// Main loop shared by both 16-bit kernels: acc[col tile][row tile] over the wave's 64 x 64 tile.
template <typename DT, bool FAST>
__device__ __forceinline__ void mfma_mainloop(const LinArgs& a, int64_t row0, int col0, int r16, int g,
                                              f32x4 (&acc)[4][4]) {
    const u16* x = static_cast<const u16*>(a.x);
    const u16* w = static_cast<const u16*>(a.w);
    const int64_t last_row = a.rows - 1;
    int64_t xr[4], wr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {   // clamp instead of branching: out-of-range tiles are never stored
        int64_t r = row0 + t * 16 + r16; xr[t] = r < last_row ? r : last_row;
        int c = col0 + t * 16 + r16; wr[t] = c < a.M - 1 ? c : a.M - 1;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int nk = (a.K + 31) / 32;
    // PF chunks of fragments in flight: a wave of this kernel has nothing else to hide the memory latency behind
    // (with one chunk ahead every 16 MFMAs waited a full round trip: 2.4 us per chunk at 16k rows x K = 384).  The
    // register sets rotate by full unrolling, never by a run-time index.
    constexpr int PF = FAST ? 4 : 1;
    s16x8 xf[PF][4], wf[PF][4];
#pragma unroll
    for (int s = 0; s < PF; ++s)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            xf[s][t] = load_frag<FAST>(x, a.ldx, xr[t], s * 32 + g * 8, a.K);       // past K: zeros, no load
            wf[s][t] = load_frag<FAST>(w, a.K, wr[t], s * 32 + g * 8, a.K);
        }
    for (int kc0 = 0; kc0 < nk; kc0 += PF) {
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            if (kc0 + s < nk) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = DT::mfma32(wf[s][i], xf[s][j], acc[i][j]);
                const int k1 = (kc0 + s + PF) * 32 + g * 8;
                if (kc0 + s + PF < nk) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        xf[s][t] = load_frag<FAST>(x, a.ldx, xr[t], k1, a.K);
                        wf[s][t] = load_frag<FAST>(w, a.K, wr[t], k1, a.K);
                    }
                }
            }
        }
    }
}

// General epilogue: any M, any strides, optional column split into a second output.
template <typename DT, int ACT, bool FAST>
__global__ __launch_bounds__(256) void linear_mfma_kernel(LinArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 128 + (wave >> 1) * 64;
    const int col0 = blockIdx.x * 128 + (wave & 1) * 64;
    if (col0 >= a.M) return;
    f32x4 acc[4][4];
    mfma_mainloop<DT, FAST>(a, row0, col0, r16, g, acc);
    const u16* res = static_cast<const u16*>(a.res);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int col = col0 + i * 16 + g * 4;   // lane holds columns col..col+3 of its rows
        if (col >= a.M) continue;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (a.bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) if (col + e < a.M) bv[e] = a.bias[col + e];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t row = row0 + j * 16 + r16;
            if (row >= a.rows) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = col + e;
                if (c >= a.M) break;
                float o = a.out_f32 ? apply_act<ACT>(acc[i][j][e] + bv[e]) : apply_act16<ACT>(acc[i][j][e] + bv[e]);
                if (res) o += DT::to_f(res[row * a.ldr + c]);
                if (a.gate && !(DT::to_f(static_cast<const u16*>(a.gate)[row * a.ldgate + c]) > 0.f)) o = 0.f;
                const bool second = a.y2 && c >= a.split;
                void* dst = second ? a.y2 : a.y;
                const int64_t off = second ? row * a.ldy2 + (c - a.split) : lin_yoff(a, row) + c;
                if (a.out_f32) static_cast<float*>(dst)[off] = o;
                else static_cast<u16*>(dst)[off] = DT::from_f(o);
            }
        }
    }
}

// Vector epilogue: M % 4 == 0, 4-element-aligned strides, no split: 8/16-byte stores.
template <typename DT, int ACT>
__global__ __launch_bounds__(256) void linear_mfma_vec_kernel(LinArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 128 + (wave >> 1) * 64;
    const int col0 = blockIdx.x * 128 + (wave & 1) * 64;
    if (col0 >= a.M) return;
    f32x4 acc[4][4];
    mfma_mainloop<DT, true>(a, row0, col0, r16, g, acc);
    const u16* res = static_cast<const u16*>(a.res);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int col = col0 + i * 16 + g * 4;
        if (col >= a.M) continue;
        float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (a.bias) bv = *reinterpret_cast<const float4*>(a.bias + col);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t row = row0 + j * 16 + r16;
            if (row >= a.rows) continue;
            float o[4] = {acc[i][j][0] + bv.x, acc[i][j][1] + bv.y, acc[i][j][2] + bv.z, acc[i][j][3] + bv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = a.out_f32 ? apply_act<ACT>(o[e]) : apply_act16<ACT>(o[e]);
            if (res) {
                uint2 rv = *reinterpret_cast<const uint2*>(res + row * a.ldr + col);
                o[0] += DT::to_f((u16)(rv.x & 0xffff)); o[1] += DT::to_f((u16)(rv.x >> 16));
                o[2] += DT::to_f((u16)(rv.y & 0xffff)); o[3] += DT::to_f((u16)(rv.y >> 16));
            }
            if (a.gate) {
                const uint2 gv = *reinterpret_cast<const uint2*>(static_cast<const u16*>(a.gate) + row * a.ldgate + col);
                if (!(DT::to_f((u16)(gv.x & 0xffff)) > 0.f)) o[0] = 0.f;
                if (!(DT::to_f((u16)(gv.x >> 16)) > 0.f)) o[1] = 0.f;
                if (!(DT::to_f((u16)(gv.y & 0xffff)) > 0.f)) o[2] = 0.f;
                if (!(DT::to_f((u16)(gv.y >> 16)) > 0.f)) o[3] = 0.f;
            }
            if (a.out_f32) {
                *reinterpret_cast<float4*>(static_cast<float*>(a.y) + lin_yoff(a, row) + col) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
                uint2 ov;
                ov.x = DT::pack2(o[0], o[1]);
                ov.y = DT::pack2(o[2], o[3]);
                *reinterpret_cast<uint2*>(static_cast<u16*>(a.y) + lin_yoff(a, row) + col) = ov;
            }
        }
    }
}

// ---- fp32: 64x64 tile, K step 16, 4x4 outputs per thread -----------------------
template <int ACT>
__global__ __launch_bounds__(256) void linear_f32_kernel(LinArgs a) {
    __shared__ float xs[16][64 + 1];
    __shared__ float ws[16][64 + 1];
    const float* x = static_cast<const float*>(a.x);
    const float* w = static_cast<const float*>(a.w);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 64;
    const int col0 = blockIdx.x * 64;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < a.K; k0 += 16) {
        for (int i = threadIdx.x; i < 64 * 16; i += 256) {
            const int r = i >> 4, k = i & 15;
            const int64_t row = row0 + r; const int col = col0 + r;
            xs[k][r] = (row < a.rows && k0 + k < a.K) ? x[row * a.ldx + k0 + k] : 0.f;
            ws[k][r] = (col < a.M && k0 + k < a.K) ? w[(int64_t)col * a.K + k0 + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            float xv[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { xv[i] = xs[k][ty * 4 + i]; wv[i] = ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xv[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
    const float* res = static_cast<const float*>(a.res);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = row0 + ty * 4 + i;
        if (row >= a.rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = col0 + tx * 4 + j;
            if (c >= a.M) continue;
            float o = apply_act<ACT>(acc[i][j] + (a.bias ? a.bias[c] : 0.f));
            if (res) o += res[row * a.ldr + c];
            if (a.gate && !(static_cast<const float*>(a.gate)[row * a.ldgate + c] > 0.f)) o = 0.f;
            if (a.y2 && c >= a.split) static_cast<float*>(a.y2)[row * a.ldy2 + (c - a.split)] = o;
            else static_cast<float*>(a.y)[lin_yoff(a, row) + c] = o;
        }
    }
}

template <typename DT>
void launch16(const LinArgs& a, int act, bool fast, bool vec, hipStream_t st) {
    dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)((a.rows + 127) / 128));
#define GO(ACT) do { \
        if (vec) hipLaunchKernelGGL((linear_mfma_vec_kernel<DT, ACT>), grid, dim3(256), 0, st, a); \
        else if (fast) hipLaunchKernelGGL((linear_mfma_kernel<DT, ACT, true>), grid, dim3(256), 0, st, a); \
        else hipLaunchKernelGGL((linear_mfma_kernel<DT, ACT, false>), grid, dim3(256), 0, st, a); } while (0)
    if (act == BSRL_ACT_RELU) GO(BSRL_ACT_RELU);
    else if (act == BSRL_ACT_GELU) GO(BSRL_ACT_GELU);
    else GO(BSRL_ACT_NONE);
#undef GO
}

int lin_dispatch(const LinArgs& a, int act, int dtype, int out_dtype, hipStream_t st, const char* what) {
    if ((a.rows + 127) / 128 > 65535 * 16) return BSRL_UNSUPPORTED;
    if (dtype == BSRL_F32) {
        dim3 grid((unsigned)((a.M + 63) / 64), (unsigned)((a.rows + 63) / 64));
        if (act == BSRL_ACT_RELU) hipLaunchKernelGGL((linear_f32_kernel<BSRL_ACT_RELU>), grid, dim3(256), 0, st, a);
        else if (act == BSRL_ACT_GELU) hipLaunchKernelGGL((linear_f32_kernel<BSRL_ACT_GELU>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((linear_f32_kernel<BSRL_ACT_NONE>), grid, dim3(256), 0, st, a);
    } else {
        const bool fast = a.K % 8 == 0 && a.ldx % 8 == 0 && bsrl_aligned(a.x, 16) && bsrl_aligned(a.w, 16);
        const int osz = out_dtype == BSRL_F32 ? 4 : 2;
        const bool vec = fast && !a.y2 && a.M % 4 == 0 && a.ldy % 4 == 0 && a.y_gstride % 4 == 0 && bsrl_aligned(a.y, 4 * osz) &&
                         (!a.bias || bsrl_aligned(a.bias, 16)) &&
                         (!a.res || (a.ldr % 4 == 0 && bsrl_aligned(a.res, 8))) &&
                         (!a.gate || (a.ldgate % 4 == 0 && bsrl_aligned(a.gate, 8)));
        if (vec && a.res && bsrl_linear_ring(a, act, dtype, st)) {
            // with a residual the ring kernel's epilogue (all residual loads of a wave tile in flight at once)
            // beats the streaming kernel at every K measured (75 vs 97 us at 128 -> 128, 150 vs 192 at 192 -> 192,
            // 475k rows)
        } else if (vec && bsrl_linear_stream(a, act, dtype, st)) {
            // many rows, modest K: the weight-resident streaming kernel
        } else if (vec && bsrl_linear_ring(a, act, dtype, st)) {
            // large, aligned, 16-bit-out problems with K a multiple of 32: operands straight into an LDS ring
        } else if (vec && bsrl_linear_tiled(a, act, dtype, st)) {
            // large, aligned, 16-bit-out problems: the LDS-tiled kernel
        } else if (dtype == BSRL_F16) launch16<F16>(a, act, fast, vec, st);
        else launch16<BF16>(a, act, fast, vec, st);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) BSRL_FAIL(BSRL_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return BSRL_OK;
}

}  // namespace

extern "C" int bsrl_linear(const void* x, int64_t ldx, const void* w, const float* bias, const void* residual,
                           int64_t ldr, void* y, int64_t ldy, void* y2, int64_t ldy2, int64_t split,
                           int64_t rows, int64_t K, int64_t M, int act, int dtype, int out_dtype,
                           bsrl_stream stream) {
    return bsrl_linear_grouped(x, ldx, w, bias, residual, ldr, y, ldy, y2, ldy2, split, rows, K, M, act, dtype, out_dtype,
                               0, 0, stream);
}

extern "C" int bsrl_linear_grouped(const void* x, int64_t ldx, const void* w, const float* bias, const void* residual,
                                   int64_t ldr, void* y, int64_t ldy, void* y2, int64_t ldy2, int64_t split,
                                   int64_t rows, int64_t K, int64_t M, int act, int dtype, int out_dtype,
                                   int64_t y_group_rows, int64_t y_group_stride, bsrl_stream stream) {
    if (!x || !w || !y) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: null pointer");
    if (rows < 0 || K <= 0 || M <= 0 || K > (1 << 20) || M > (1 << 20))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: bad shape rows=%lld K=%lld M=%lld", (long long)rows, (long long)K, (long long)M);
    if (ldx < K || ldy < (y2 ? split : M) || (residual && ldr < M))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: row stride smaller than row");
    if (y2 && (split <= 0 || split >= M || ldy2 < M - split)) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: bad split");
    if (act < 0 || act > 2) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: bad act %d", act);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: bad dtype");
    if (out_dtype != dtype && out_dtype != BSRL_F32) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear: out_dtype must be dtype or F32");
    if (y_group_rows < 0 || (y_group_rows > 0 && (y2 || rows % y_group_rows != 0 || y_group_rows > (1 << 20) ||
                                                  y_group_stride < y_group_rows * ldy)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_linear_grouped: groups need rows %% group == 0, group stride >= group * ldy, no split");
    if (rows == 0) return BSRL_OK;
    LinArgs a{x, ldx, w, bias, residual, ldr, y, ldy, y2, ldy2, split, rows, (int)K, (int)M, out_dtype == BSRL_F32,
              (int)y_group_rows, y_group_stride, nullptr, 0};
    return lin_dispatch(a, act, dtype, out_dtype, static_cast<hipStream_t>(stream), "bsrl_linear");
}

extern "C" int bsrl_mlp2(const void* x, int64_t ldx, const void* w1, const float* b1, int64_t K1, const void* w2,
                         const float* b2, void* y, int64_t ldy, int64_t rows, int64_t d, int dtype, int64_t y_group_rows,
                         int64_t y_group_stride, bsrl_stream stream) {
    if (!x || !w1 || !b1 || !w2 || !b2 || !y) BSRL_FAIL(BSRL_EINVAL, "bsrl_mlp2: null pointer");
    if (rows < 0 || K1 <= 0 || d <= 0 || K1 > (1 << 20) || d > (1 << 20))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_mlp2: bad shape rows=%lld K1=%lld d=%lld", (long long)rows, (long long)K1, (long long)d);
    if (ldx < K1 || ldy < d) BSRL_FAIL(BSRL_EINVAL, "bsrl_mlp2: row stride smaller than row");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_mlp2: bad dtype");
    if (y_group_rows < 0 || (y_group_rows > 0 && (rows % y_group_rows != 0 || y_group_rows > (1 << 20) || y_group_stride < y_group_rows * ldy)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_mlp2: groups need rows %% group == 0 and group stride >= group * ldy");
    if (dtype == BSRL_F32) return BSRL_UNSUPPORTED;
    if (rows == 0) return BSRL_OK;
    LinArgs l2{nullptr, 0, w2, b2, nullptr, 0, y, ldy, nullptr, 0, 0, rows, (int)d, (int)d, 0, (int)y_group_rows, y_group_stride, nullptr, 0};
    if (!bsrl_mlp2_stream(l2, x, ldx, w1, b1, K1, dtype, static_cast<hipStream_t>(stream))) return BSRL_UNSUPPORTED;
    BSRL_CHECK_LAUNCH("bsrl_mlp2");
    return BSRL_OK;
}

extern "C" int bsrl_linear_gated(const void* x, int64_t ldx, const void* w, const void* gate, int64_t ldgate,
                                 void* y, int64_t ldy, int64_t rows, int64_t K, int64_t M, int dtype,
                                 bsrl_stream stream) {
    if (!x || !w || !y || !gate) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear_gated: null pointer");
    if (rows < 0 || K <= 0 || M <= 0 || K > (1 << 20) || M > (1 << 20))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_linear_gated: bad shape rows=%lld K=%lld M=%lld", (long long)rows, (long long)K, (long long)M);
    if (ldx < K || ldy < M || ldgate < M) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear_gated: row stride smaller than row");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_linear_gated: bad dtype");
    if (rows == 0) return BSRL_OK;
    LinArgs a{x, ldx, w, nullptr, nullptr, 0, y, ldy, nullptr, 0, 0, rows, (int)K, (int)M, 0, 0, 0, gate, ldgate};
    return lin_dispatch(a, BSRL_ACT_NONE, dtype, dtype, static_cast<hipStream_t>(stream), "bsrl_linear_gated");
}
