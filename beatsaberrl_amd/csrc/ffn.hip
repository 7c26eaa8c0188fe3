// Fused FFN for gfx950:  xo = x + act(h2 W0^T + b0) W2^T + b2 ;  ho = LayerNorm(xo).
//
// A workgroup of 4 waves owns 64*RT rows; each wave keeps its 16*RT-row slice
// of the fp32 output accumulator (residual + b2 folded in) and its h2 operand
// fragments in registers for the whole kernel.  The hidden layer is walked in
// chunks of 32 units: the chunk's W0 rows and W2 columns are staged once per
// workgroup in LDS (two buffers; the next chunk is loaded into registers one
// chunk ahead and parked while the current one is consumed, one barrier per
// chunk) in MFMA fragment order (W0 in plain k order - it meets h2
// as loaded from memory; W2 in the order in which the up-projection's
// accumulator tiles pack into an operand: k = 4g..4g+3 then 16+4g..16+4g+3 for
// lane group g), the up-projection runs on the matrix cores, bias + activation
// + the single rounding to the 16-bit type happen in registers, and the
// down-projection accumulates straight onto the residual.  The hidden
// activation (R x F) never reaches memory.
//
// Rounding points follow the reference kernel (python/beat_arena_env/csrc/
// fused_ffn.cu:42-59): fp32 accumulate in both GEMMs, hidden = act(S + b0)
// rounded once, xo = round(x + (O + b2)), LayerNorm statistics on the ROUNDED
// xo, ho rounded once.  A row's result depends only on that row and the
// weights (fixed k order, no atomics), whatever R is.
// Replaces fp16_gemm.ffn_fused (fused_ffn.cu:242-485, 551-619).
#include "bsrl_common.h"

namespace {

struct FfnArgs {
    const u16 *x, *h2, *w0, *w2;
    const float *b0, *b2, *ln_w, *ln_b;
    u16 *xo, *ho;
    int64_t rows; int F; float eps;
};

template <typename DT> __device__ __forceinline__ uint32_t pk2(float a, float b) {
    return DT::pack2(a, b);
}

template <typename DT, int D, int RT, int ACT>
__global__ __launch_bounds__(256, (RT * D <= 384) ? 2 : 1) void ffn_fused_kernel(FfnArgs a) {
    constexpr int NT = D / 16, KC = D / 32, NFR = 2 * KC + NT;
    constexpr int PER = (NFR + 3) / 4;             // fragments each wave stages per chunk
    extern __shared__ uint4 wl_all[];              // 2 x NFR fragments: chunk ch lives in buffer ch & 1
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * (RT * 16);

    // one chunk's weight fragments, straight from the nn.Linear layouts: W0 rows in plain k order,
    // W2 columns in the accumulator-pack order (4g..4g+3, 16+4g..16+4g+3)
    uint4 pre[PER];
    auto gload = [&](int ch) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = wave + 4 * i;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (f < 2 * KC) {
                const int ntl = f / KC, c = f % KC;
                v = *reinterpret_cast<const uint4*>(a.w0 + (int64_t)(32 * ch + 16 * ntl + r16) * D + 32 * c + 8 * g);
            } else if (f < NFR) {
                const u16* p = a.w2 + (int64_t)(16 * (f - 2 * KC) + r16) * a.F + 32 * ch + 4 * g;
                const uint2 lo = *reinterpret_cast<const uint2*>(p), hi = *reinterpret_cast<const uint2*>(p + 16);
                v = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
            pre[i] = v;
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = wave + 4 * i;
            if (f < NFR) wl_all[(buf * NFR + f) * 64 + lane] = pre[i];
        }
    };
    const int nch = a.F / 32;
    gload(0);

    f32x4 xa[RT][NT];
    union { s16x8 v; uint4 u; uint32_t w[4]; } hf[RT][KC];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        int64_t row = row0 + rt * 16 + r16; row = row < a.rows ? row : a.rows - 1;
#pragma unroll
        for (int c = 0; c < KC; ++c) hf[rt][c].u = *reinterpret_cast<const uint4*>(a.h2 + row * D + 32 * c + 8 * g);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint2 xv = *reinterpret_cast<const uint2*>(a.x + row * D + 16 * nt + 4 * g);
            const float4 b = *reinterpret_cast<const float4*>(a.b2 + 16 * nt + 4 * g);
            xa[rt][nt] = (f32x4){DT::to_f((u16)(xv.x & 0xffff)) + b.x, DT::to_f((u16)(xv.x >> 16)) + b.y,
                                 DT::to_f((u16)(xv.y & 0xffff)) + b.z, DT::to_f((u16)(xv.y >> 16)) + b.w};
        }
    }
    lstore(0);
    if (nch > 1) gload(1);
    for (int ch = 0; ch < nch; ++ch) {
        const uint4* wl = wl_all + (ch & 1) * NFR * 64;
        __syncthreads();        // chunk ch is complete in buffer ch & 1; buffer (ch + 1) & 1 is no longer read
        if (ch + 1 < nch) {
            lstore((ch + 1) & 1);                  // chunk ch + 1 (loaded one chunk ago) -> the free buffer
            if (ch + 2 < nch) gload(ch + 2);       // in flight during this chunk's MFMAs
        }
        f32x4 acc[2][RT];
#pragma unroll
        for (int ntl = 0; ntl < 2; ++ntl) {
            const float4 b = *reinterpret_cast<const float4*>(a.b0 + 32 * ch + 16 * ntl + 4 * g);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) acc[ntl][rt] = (f32x4){b.x, b.y, b.z, b.w};
        }
#pragma unroll
        for (int c = 0; c < KC; ++c)
#pragma unroll
            for (int ntl = 0; ntl < 2; ++ntl) {
                const s16x8 w = __builtin_bit_cast(s16x8, wl[(ntl * KC + c) * 64 + lane]);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) acc[ntl][rt] = DT::mfma32(w, hf[rt][c].v, acc[ntl][rt]);
            }
        union { s16x8 v; uint32_t w[4]; } hid[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int ntl = 0; ntl < 2; ++ntl) {
                hid[rt].w[ntl * 2] = pk2<DT>(apply_act16<ACT>(acc[ntl][rt][0]), apply_act16<ACT>(acc[ntl][rt][1]));
                hid[rt].w[ntl * 2 + 1] = pk2<DT>(apply_act16<ACT>(acc[ntl][rt][2]), apply_act16<ACT>(acc[ntl][rt][3]));
            }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const s16x8 w = __builtin_bit_cast(s16x8, wl[(2 * KC + nt) * 64 + lane]);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) xa[rt][nt] = DT::mfma32(w, hid[rt].v, xa[rt][nt]);
        }
    }
    // epilogue: round, store, optional LayerNorm on the rounded row
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int64_t row = row0 + rt * 16 + r16;
        const bool live = row < a.rows;
        float s = 0.f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t lo = pk2<DT>(xa[rt][nt][0], xa[rt][nt][1]), hi = pk2<DT>(xa[rt][nt][2], xa[rt][nt][3]);
            if (live) *reinterpret_cast<uint2*>(a.xo + row * D + 16 * nt + 4 * g) = make_uint2(lo, hi);
            xa[rt][nt] = (f32x4){DT::to_f((u16)(lo & 0xffff)), DT::to_f((u16)(lo >> 16)),
                                 DT::to_f((u16)(hi & 0xffff)), DT::to_f((u16)(hi >> 16))};
            s += (xa[rt][nt][0] + xa[rt][nt][1]) + (xa[rt][nt][2] + xa[rt][nt][3]);
        }
        if (a.ho) {
            s += __shfl_xor(s, 16, WAVE); s += __shfl_xor(s, 32, WAVE);
            const float mean = s * (1.0f / D);
            float q = 0.f;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) { const float t = xa[rt][nt][i] - mean; q = fmaf(t, t, q); }
            q += __shfl_xor(q, 16, WAVE); q += __shfl_xor(q, 32, WAVE);
            const float rstd = 1.0f / sqrtf(q * (1.0f / D) + a.eps);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 gm = *reinterpret_cast<const float4*>(a.ln_w + 16 * nt + 4 * g);
                const float4 bt = *reinterpret_cast<const float4*>(a.ln_b + 16 * nt + 4 * g);
                const uint32_t lo = pk2<DT>((xa[rt][nt][0] - mean) * rstd * gm.x + bt.x, (xa[rt][nt][1] - mean) * rstd * gm.y + bt.y);
                const uint32_t hi = pk2<DT>((xa[rt][nt][2] - mean) * rstd * gm.z + bt.z, (xa[rt][nt][3] - mean) * rstd * gm.w + bt.w);
                if (live) *reinterpret_cast<uint2*>(a.ho + row * D + 16 * nt + 4 * g) = make_uint2(lo, hi);
            }
        }
    }
}

template <typename DT, int D, int RT, int ACT>
bool launch_act(const FfnArgs& a, hipStream_t st) {
    constexpr size_t lds = 2 * (size_t)(D / 8) * 64 * sizeof(uint4);       // two chunk buffers
    auto kern = ffn_fused_kernel<DT, D, RT, ACT>;
    if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return false;
    const unsigned grid = (unsigned)((a.rows + 64 * RT - 1) / (64 * RT));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, a);
    return true;
}
template <typename DT, int D, int RT>
bool launch(const FfnArgs& a, int act, hipStream_t st) {
    if (act == BSRL_ACT_RELU) return launch_act<DT, D, RT, BSRL_ACT_RELU>(a, st);
    if (act == BSRL_ACT_GELU) return launch_act<DT, D, RT, BSRL_ACT_GELU>(a, st);
    return launch_act<DT, D, RT, BSRL_ACT_NONE>(a, st);
}

template <typename DT>
bool dispatch(const FfnArgs& a, int64_t d, int act, hipStream_t st) {
    if (d == 128) return launch<DT, 128, 2>(a, act, st);
    if (d == 192) return launch<DT, 192, 2>(a, act, st);
    if (d == 256) return launch<DT, 256, 2>(a, act, st);
    return launch<DT, 384, 1>(a, act, st);
}

}  // namespace

extern "C" int bsrl_ffn_fused_supported(int64_t d, int64_t F, int dtype) {
    return (d == 128 || d == 192 || d == 256 || d == 384) && F > 0 && F % 32 == 0 &&
           (dtype == BSRL_F16 || dtype == BSRL_BF16);
}

extern "C" int bsrl_ffn_fused(const void* x, const void* h2, const void* w0, const float* b0, const void* w2,
                              const float* b2, const float* ln_w, const float* ln_b, float eps, void* xo, void* ho,
                              int64_t rows, int64_t d, int64_t F, int act, int dtype, bsrl_stream stream) {
    if (!x || !h2 || !w0 || !b0 || !w2 || !b2 || !xo) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_fused: null pointer");
    if ((ln_w == nullptr) != (ho == nullptr) || (ln_w == nullptr) != (ln_b == nullptr))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_fused: ln_w, ln_b and ho go together");
    if (rows < 0 || d <= 0 || F <= 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_fused: bad shape");
    if (act < 0 || act > 2) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_fused: bad act %d", act);
    if (!bsrl_ffn_fused_supported(d, F, dtype)) return BSRL_UNSUPPORTED;
    const void* ptrs[] = {x, h2, w0, w2, xo, ho, b0, b2, ln_w, ln_b};
    for (const void* p : ptrs) if (p && !bsrl_aligned(p, 16)) return BSRL_UNSUPPORTED;
    if (rows == 0) return BSRL_OK;
    FfnArgs a{static_cast<const u16*>(x), static_cast<const u16*>(h2), static_cast<const u16*>(w0),
              static_cast<const u16*>(w2), b0, b2, ln_w, ln_b, static_cast<u16*>(xo), static_cast<u16*>(ho),
              rows, (int)F, eps};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool ok = dtype == BSRL_F16 ? dispatch<F16>(a, d, act, st) : dispatch<BF16>(a, d, act, st);
    if (!ok) return BSRL_UNSUPPORTED;
    BSRL_CHECK_LAUNCH("bsrl_ffn_fused");
    return BSRL_OK;
}
