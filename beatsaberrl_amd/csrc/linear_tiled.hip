// LDS-tiled MFMA linear for large row counts: y = act(x W^T + b) (+ residual), 16-bit in / out.
//
// Workgroup tile 256 rows x 128 columns, K walked in steps of 64 through LDS.  All 256
// threads load the step's x (256 x 64) and W (128 x 64) tiles with 16-byte global loads one
// step ahead into registers and park them in LDS in MFMA fragment order (fragment = 64
// lanes x 16 B, one ds_read_b128 per operand).  Inside a fragment the 16-byte slot of lane l
// is l ^ (2 * (l / 16) + k chunk): the XOR keeps the slots of any 8 consecutive lanes distinct
// modulo 8 for the reads AND for the loader's writes (8 consecutive loader threads hold the
// 8 k pieces of one row, which land in lanes r, r + 16, r + 32, r + 48 of two fragments -
// unswizzled, all on the same 4 banks); wave w owns rows
// [64w, 64w + 64) x all 128 columns: 4 x 8 accumulator tiles, 64 MFMAs per step against 24
// fragment reads.  x and y cross HBM exactly once per column block and in full 128-byte
// rows: the epilogue adds bias, applies the activation, then transposes each wave's
// accumulators through LDS in fp32 so that 16 lanes write (and read the residual of) one
// 256-byte row segment; the sum is rounded once.
//
// Same arithmetic contract as the direct-from-global kernel in linear.hip (fp32 accumulate,
// fixed k order, a row's result independent of the batch) - the two are interchangeable and
// the entry point picks by shape.
#include "linear_args.h"

namespace {

constexpr int BM = 256, BN = 128, BK = 64;
constexpr int KCH = BK / 32;                       // 32-wide k chunks per step
constexpr int XF = (BM / 16) * KCH;                // x fragments per step (32)
constexpr int WF = (BN / 16) * KCH;                // W fragments per step (16)
constexpr int LDS_U4 = (XF + WF) * 64;             // 48 KB
constexpr int EP_LD = BN + 4;                      // epilogue row pitch (floats)

template <typename DT, int ACT>
__global__ __launch_bounds__(256, 2) void linear_tiled_kernel(LinArgs a) {
    __shared__ uint4 lds[LDS_U4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * BM;
    const int col0 = blockIdx.x * BN;
    const u16* x = static_cast<const u16*>(a.x);
    const u16* w = static_cast<const u16*>(a.w);
    const int K = a.K;

    // loader mapping: a thread owns the 16-byte piece (row, 8 k) = (tid / 8 + 32 j, 8 * (tid % 8))
    const int lq = tid & 7, lr = tid >> 3;         // k piece 0..7, row 0..31
    int64_t xrow[8]; int wrow[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) { int64_t r = row0 + lr + 32 * j; xrow[j] = (r < a.rows ? r : a.rows - 1) * a.ldx; }
#pragma unroll
    for (int j = 0; j < 4; ++j) { int c = col0 + lr + 32 * j; wrow[j] = (c < a.M ? c : a.M - 1) * K; }
    // where that piece lives in LDS: fragment (row tile, k chunk), lane (row % 16) + 16 * (piece % 4)
    const int kc_of = lq >> 2;
    const int frag_lane = ((lr & 15) + 16 * (lq & 3)) ^ (2 * (lq & 3) + kc_of);     // swizzled slot
    uint4 xr[8], wr[4];
    auto gload = [&](int k0) {
        const int k = k0 + 8 * lq;
        const bool on = k < K;
#pragma unroll
        for (int j = 0; j < 8; ++j) xr[j] = on ? *reinterpret_cast<const uint4*>(x + xrow[j] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) wr[j] = on ? *reinterpret_cast<const uint4*>(w + wrow[j] + k) : make_uint4(0, 0, 0, 0);
    };
    auto lstore = [&]() {
#pragma unroll
        for (int j = 0; j < 8; ++j) lds[(((lr >> 4) + 2 * j) * KCH + kc_of) * 64 + frag_lane] = xr[j];
#pragma unroll
        for (int j = 0; j < 4; ++j) lds[(XF + ((lr >> 4) + 2 * j) * KCH + kc_of) * 64 + frag_lane] = wr[j];
    };

    f32x4 acc[8][4];                               // [column tile][row tile]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int nsteps = (K + BK - 1) / BK;
    gload(0);
    for (int s = 0; s < nsteps; ++s) {
        __syncthreads();                           // the previous step's fragments are no longer read
        lstore();
        __syncthreads();
        if (s + 1 < nsteps) gload((s + 1) * BK);   // in flight during this step's MFMAs
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
            s16x8 xf[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) xf[j] = __builtin_bit_cast(s16x8, lds[((wave * 4 + j) * KCH + c) * 64 + (lane ^ (2 * g + c))]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const s16x8 wf = __builtin_bit_cast(s16x8, lds[(XF + i * KCH + c) * 64 + (lane ^ (2 * g + c))]);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = DT::mfma32(wf, xf[j], acc[i][j]);
            }
        }
    }
    __syncthreads();                               // operand tiles dead: LDS becomes the epilogue staging area

    // epilogue: per wave, 16 rows at a time through a private fp32 [16][BN + 4] region
    float* ep = reinterpret_cast<float*>(lds) + wave * (16 * EP_LD);
    const u16* res = static_cast<const u16*>(a.res);
    u16* y = static_cast<u16*>(a.y);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int col = col0 + i * 16 + 4 * g;
            float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
            if (a.bias && col < a.M) b = *reinterpret_cast<const float4*>(a.bias + col);
            const float4 o = make_float4(apply_act16<ACT>(acc[i][j][0] + b.x), apply_act16<ACT>(acc[i][j][1] + b.y),
                                         apply_act16<ACT>(acc[i][j][2] + b.z), apply_act16<ACT>(acc[i][j][3] + b.w));
            *reinterpret_cast<float4*>(ep + r16 * EP_LD + i * 16 + 4 * g) = o;
        }
        // lane -> (row = lane / 16 + 4 q, 4 columns at 4 m and 4 at 64 + 4 m, m = lane % 16): consecutive lanes read
        // consecutive 16-byte slots of the staging row (no bank conflict) and 16 lanes write one 128-byte row segment
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int rl = (lane >> 4) + 4 * q, c4 = 4 * (lane & 15);
            const int64_t row = row0 + wave * 64 + j * 16 + rl;
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int col = col0 + 64 * hh + c4;
                const float4 f = *reinterpret_cast<const float4*>(ep + rl * EP_LD + 64 * hh + c4);
                float v[4] = {f.x, f.y, f.z, f.w};
                if (row < a.rows && col < a.M) {
                    if (res) {
                        const uint2 rv = *reinterpret_cast<const uint2*>(res + row * a.ldr + col);
                        v[0] += DT::to_f((u16)(rv.x & 0xffff)); v[1] += DT::to_f((u16)(rv.x >> 16));
                        v[2] += DT::to_f((u16)(rv.y & 0xffff)); v[3] += DT::to_f((u16)(rv.y >> 16));
                    }
                    if (a.gate) {
                        const uint2 gv = *reinterpret_cast<const uint2*>(static_cast<const u16*>(a.gate) + row * a.ldgate + col);
                        if (!(DT::to_f((u16)(gv.x & 0xffff)) > 0.f)) v[0] = 0.f;
                        if (!(DT::to_f((u16)(gv.x >> 16)) > 0.f)) v[1] = 0.f;
                        if (!(DT::to_f((u16)(gv.y & 0xffff)) > 0.f)) v[2] = 0.f;
                        if (!(DT::to_f((u16)(gv.y >> 16)) > 0.f)) v[3] = 0.f;
                    }
                    uint2 ov;
                    ov.x = DT::pack2(v[0], v[1]);
                    ov.y = DT::pack2(v[2], v[3]);
                    *reinterpret_cast<uint2*>(y + lin_yoff(a, row) + col) = ov;
                }
            }
        }
    }
}

template <typename DT>
void launch(const LinArgs& a, int act, hipStream_t st) {
    dim3 grid((unsigned)((a.M + BN - 1) / BN), (unsigned)((a.rows + BM - 1) / BM));
    if (act == BSRL_ACT_RELU) hipLaunchKernelGGL((linear_tiled_kernel<DT, BSRL_ACT_RELU>), grid, dim3(256), 0, st, a);
    else if (act == BSRL_ACT_GELU) hipLaunchKernelGGL((linear_tiled_kernel<DT, BSRL_ACT_GELU>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((linear_tiled_kernel<DT, BSRL_ACT_NONE>), grid, dim3(256), 0, st, a);
}

}  // namespace

bool bsrl_linear_tiled(const LinArgs& a, int act, int dtype, hipStream_t st) {
    static_assert(16 * EP_LD * 4 * 4 <= LDS_U4 * 16, "epilogue staging must fit in the operand tiles");
    // worth it only when there are enough rows to fill the chip with 256-row tiles
    if (a.out_f32 || a.y2 || a.rows < 4096 || a.M % 8 != 0 || a.K % 8 != 0) return false;
    if (a.ldy % 8 != 0 || a.y_gstride % 8 != 0 || !bsrl_aligned(a.y, 16) || (a.res && (a.ldr % 8 != 0 || !bsrl_aligned(a.res, 16)))) return false;
    if (a.gate && (a.ldgate % 4 != 0 || !bsrl_aligned(a.gate, 8))) return false;
    if ((a.rows + BM - 1) / BM > 65535) return false;
    if (dtype == BSRL_F16) launch<F16>(a, act, st);
    else launch<BF16>(a, act, st);
    return true;
}
