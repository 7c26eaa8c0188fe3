// One-query attention pool of the adapool critic without materialising keys and values.
//
// The reference's critic (python/policy.py:1346-1403) projects k = Wk hv + bk and v = Wv hv + bv for ALL T tokens of
// every env (a (B T, d) -> (B T, 2d) GEMM, ~3 % of the forward's MACs and a 2 (B T d) write + read) and then attends
// with ONE query per env.  With a single query the projections commute with the pool:
//     q_h . k_j = (Wk_h^T q_h) . hv_j + q_h . bk_h          the last term is one constant per (env, head): it cancels
//                                                            in the softmax over j
//     sum_j p_j v_j = Wv_h (sum_j p_j hv_j) + bv_h          because sum_j p_j = 1
// so this kernel takes qk[b, h, :] = Wk_h^T q_h (a (B, d) -> (B, H d) GEMM on B rows), computes
//     hv_j = LayerNorm(x_res[b, j]) rounded to the stream dtype, as the reference's critic_ln output is
//     p[h] = softmax_j(hv_j . qk[b, h] / sqrt(dh) + key_bias[b, j])           (fp32; masked keys get exactly 0)
//     pooled[b, h, :] = sum_j p[h][j] hv_j                                     (p rounded to the stream dtype for the
//                                                                               matrix product, as attention does)
// and the caller finishes a_h = Wv_h pooled_h + bv_h with one more GEMM on B rows.  x_res is read once; nothing of
// size (B T, d) is written.  Same result as the reference's order up to rounding (k and v are never rounded here).
//
// One wave per env (T <= 32, H <= 16, 16-bit streams), four envs per workgroup.
//   1. the env's contiguous T x d block goes to LDS with coalesced 16-byte loads (rows T..31 zero);
//   2. LayerNorm with two lanes per row: a lane keeps its half row in registers (fp32) through mean, centred variance and
//      the affine map, and writes the rounded half row back in place;
//   3. scores as MFMAs: D[token][head] = hv (A: 16 tokens x 32 k, plain row reads) x qk (B: lanes head < H, straight from
//      global memory); lane (head, g) ends with that head's scores of tokens 16 t + 4 g + e: the softmax is an in-lane
//      reduction plus two cross-lane steps, all heads at once;
//   4. pool as MFMAs over the token index: D[column][head] = hv^T x p.  The contraction slot (g, j) of a lane stands for
//      token 4 g + j (j < 4) or 16 + 4 g + (j - 4): that is exactly what the lane holds after step 3, so p needs no
//      transpose, and hv^T comes out of LDS through the transpose load with the same token order.
// A first version on the vector ALU alone (dot products by butterfly or in-lane) took 330 - 390 us at B = 16384, as
// long as the three kernels it replaced: ~4000 VALU instructions per env against ~1000 here.
#include "bsrl_common.h"

namespace {

constexpr int CP_ROWS = 32;

struct CpArgs {
    const u16* x; const float* w; const float* b; float eps; const u16* qk; const u16* key_bias; u16* pooled;
    int64_t B; int T, H; float scale;
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4v __attribute__((ext_vector_type(4)));

template <typename DT, int D>
__global__ __launch_bounds__(256) void critic_pool_kernel(CpArgs a) {
    constexpr int PITCH = D + 8;                           // elements: rows 16 B apart modulo 128 B
    constexpr int HALF = D / 2, NCH = HALF / 8;            // a lane's half row: NCH 16-byte chunks
    constexpr int PPR = D / 8;                             // 16-byte pieces per row
    constexpr int KC = D / 32;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n16 = lane & 15, g = lane >> 4;
    const int T = a.T, H = a.H;
    // workgroup-shared: LayerNorm weight and bias (fp32)
    float* lw = reinterpret_cast<float*>(smem);
    float* lb = lw + D;
    for (int i = tid; i < D; i += 256) { lw[i] = a.w[i]; lb[i] = a.b[i]; }
    __syncthreads();                                        // the only workgroup barrier
    const int64_t env = (int64_t)blockIdx.x * 4 + wave;
    if (env >= a.B) return;
    u16* rows = reinterpret_cast<u16*>(smem + 2 * D * sizeof(float)) + wave * (CP_ROWS * PITCH + 2 * CP_ROWS);
    float* kb = reinterpret_cast<float*>(rows + CP_ROWS * PITCH);          // key bias per token (fp32, -inf = masked)
    const u16* xe = a.x + env * (int64_t)T * D;

    // the query side first (its latency hides behind steps 1 and 2): B fragments of qk, lanes head < H
    u32x4 qf[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        qf[c] = (u32x4){0u, 0u, 0u, 0u};
        if (n16 < H) qf[c] = *reinterpret_cast<const u32x4*>(a.qk + (env * H + n16) * (int64_t)D + 32 * c + 8 * g);
    }
    // 1. rows to LDS, four loads in flight per lane
    {
        const int npieces = T * PPR;
        for (int p0 = lane; p0 < npieces; p0 += 4 * WAVE) {
            u32x4 r[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) if (p0 + u * WAVE < npieces) r[u] = *reinterpret_cast<const u32x4*>(xe + (int64_t)(p0 + u * WAVE) * 8);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int p = p0 + u * WAVE;
                if (p < npieces) *reinterpret_cast<u32x4*>(rows + (p / PPR) * PITCH + (p % PPR) * 8) = r[u];
            }
        }
        for (int p = T * PPR + lane; p < CP_ROWS * PPR; p += WAVE)
            *reinterpret_cast<u32x4*>(rows + (p / PPR) * PITCH + (p % PPR) * 8) = (u32x4){0u, 0u, 0u, 0u};
        if (lane < CP_ROWS) {
            float t = -INFINITY;
            if (lane < T) {
                t = 0.f;
                if (a.key_bias) {
                    const float v = DT::to_f(a.key_bias[env * T + lane]);
                    t = v < -0.5f * BSRL_MASK_BIAS ? -INFINITY : v;
                }
            }
            kb[lane] = t;
        }
    }
    asm volatile("" ::: "memory");                          // LDS is private to the wave from here: program order is enough
    // 2. LayerNorm, lane = (row lane / 2, half lane % 2)
    {
        const int row = lane >> 1, half = lane & 1;
        u16* rp = rows + row * PITCH + half * HALF;
        float v[HALF];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const u32x4 r = *reinterpret_cast<const u32x4*>(rp + 8 * c);
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[8 * c + 2 * e] = DT::to_f((u16)(r[e] & 0xffff)); v[8 * c + 2 * e + 1] = DT::to_f((u16)(r[e] >> 16)); }
        }
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < HALF; ++e) s += v[e];
        s += __shfl_xor(s, 1, WAVE);
        const float mean = s * (1.0f / D);
        float q = 0.f;
#pragma unroll
        for (int e = 0; e < HALF; ++e) { const float t = v[e] - mean; q = fmaf(t, t, q); }
        q += __shfl_xor(q, 1, WAVE);
        const float rstd = 1.0f / sqrtf(q * (1.0f / D) + a.eps);
        if (row < T) {                                      // rows T..31 stay zero
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const float4 w0 = *reinterpret_cast<const float4*>(lw + half * HALF + 8 * c), w1 = *reinterpret_cast<const float4*>(lw + half * HALF + 8 * c + 4);
                const float4 b0 = *reinterpret_cast<const float4*>(lb + half * HALF + 8 * c), b1 = *reinterpret_cast<const float4*>(lb + half * HALF + 8 * c + 4);
                const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                const float bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float o0 = (v[8 * c + 2 * e] - mean) * rstd * wv[2 * e] + bv[2 * e];
                    const float o1 = (v[8 * c + 2 * e + 1] - mean) * rstd * wv[2 * e + 1] + bv[2 * e + 1];
                    o[e] = DT::pack2(o0, o1);
                }
                *reinterpret_cast<u32x4*>(rp + 8 * c) = o;
            }
        }
    }
    asm volatile("" ::: "memory");
    // 3. scores: D[m = token 16 t + 4 g' + e][n = head], lane (n16, g') holds tokens 16 t + 4 g + e of head n16
    f32x4 sc[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int c = 0; c < KC; ++c) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const u32x4 hf = *reinterpret_cast<const u32x4*>(rows + (16 * t + n16) * PITCH + 32 * c + 8 * g);
            sc[t] = DT::mfma32(__builtin_bit_cast(s16x8, hf), __builtin_bit_cast(s16x8, qf[c]), sc[t]);
        }
    }
    // softmax over the 32 token slots of each head: 8 in the lane, then lanes n16 + 16 g
    float p[8];
    float m = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) { p[4 * t + e] = sc[t][e] * a.scale + kb[16 * t + 4 * g + e]; m = fmaxf(m, p[4 * t + e]); }
    m = fmaxf(m, __shfl_xor(m, 16, WAVE));
    m = fmaxf(m, __shfl_xor(m, 32, WAVE));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) { p[j] = __expf(p[j] - m); sum += p[j]; }      // token 0 (the lead) is never masked: m is finite
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    const float inv = 1.0f / sum;
    u32x4 pf;                                               // B fragment of the pool: slot (g, j) = token 4 g + j | 16 + 4 g + (j - 4)
#pragma unroll
    for (int e = 0; e < 4; ++e) pf[e] = DT::pack2(p[2 * e] * inv, p[2 * e + 1] * inv);
    if (n16 >= H) pf = (u32x4){0u, 0u, 0u, 0u};
    // 4. pool: D[m = column 16 j + 4 g' + e][n = head]; A = hv^T through the transpose load, rows in the slot order above
    u16* out = a.pooled + (env * H + n16) * (int64_t)D;
    typedef __attribute__((address_space(3))) s16x4v* lptr;
#pragma unroll
    for (int j = 0; j < D / 16; ++j) {
        const u16* tp = rows + (4 * g + (n16 >> 2)) * PITCH + 16 * j + 4 * (n16 & 3);
        const s16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(tp));
        const s16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(tp + 16 * PITCH));
        const s16x8 af = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const f32x4 o = DT::mfma32(af, __builtin_bit_cast(s16x8, pf), (f32x4){0.f, 0.f, 0.f, 0.f});
        if (n16 < H) {
            u32x2 ov;
            ov[0] = DT::pack2(o[0], o[1]);
            ov[1] = DT::pack2(o[2], o[3]);
            *reinterpret_cast<u32x2*>(out + 16 * j + 4 * g) = ov;
        }
    }
}

template <typename DT, int D>
int launch(const CpArgs& a, hipStream_t st) {
    const size_t lds = 2 * D * sizeof(float) + 4 * ((size_t)CP_ROWS * (D + 8) * sizeof(u16) + 2 * CP_ROWS * sizeof(u16));
    auto kern = critic_pool_kernel<DT, D>;
    if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return BSRL_UNSUPPORTED;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)((a.B + 3) / 4)), dim3(256), lds, st, a);
    return BSRL_OK;
}

template <typename DT>
int by_d(const CpArgs& a, int d, hipStream_t st) {
    switch (d) {
        case 128: return launch<DT, 128>(a, st);
        case 192: return launch<DT, 192>(a, st);
        case 256: return launch<DT, 256>(a, st);
        default: return BSRL_UNSUPPORTED;
    }
}

}  // namespace

extern "C" int bsrl_critic_pool(const void* x_res, const float* ln_weight, const float* ln_bias, float eps, const void* qk,
                                const void* key_bias, void* pooled, int64_t B, int64_t T, int64_t d, int64_t H, int dtype,
                                bsrl_stream stream) {
    if (!x_res || !ln_weight || !ln_bias || !qk || !pooled) BSRL_FAIL(BSRL_EINVAL, "bsrl_critic_pool: null pointer");
    if (B < 0 || T < 1 || d < 1 || H < 1 || d % H != 0)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_critic_pool: bad shape B=%lld T=%lld d=%lld H=%lld", (long long)B, (long long)T, (long long)d, (long long)H);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_critic_pool: bad dtype %d", dtype);
    if (dtype == BSRL_F32 || T > CP_ROWS || H > 16 || (d != 128 && d != 192 && d != 256)) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(x_res, 16) || !bsrl_aligned(qk, 16) || !bsrl_aligned(pooled, 8)) return BSRL_UNSUPPORTED;
    if (B == 0) return BSRL_OK;
    if ((B + 3) / 4 > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_critic_pool: too many envs");
    CpArgs a{static_cast<const u16*>(x_res), ln_weight, ln_bias, eps, static_cast<const u16*>(qk),
             static_cast<const u16*>(key_bias), static_cast<u16*>(pooled), B, (int)T, (int)H, (float)(1.0 / sqrt((double)(d / H)))};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rc = dtype == BSRL_F16 ? by_d<F16>(a, (int)d, st) : by_d<BF16>(a, (int)d, st);
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH("bsrl_critic_pool");
    return BSRL_OK;
}
