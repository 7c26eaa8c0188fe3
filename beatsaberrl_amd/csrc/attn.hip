// Short-sequence masked multi-head attention (T <= 48 keys) for gfx950.
//
// 16-bit path: one wave64 per (env, head); a workgroup is the H heads of one env where the shape allows (second kernel
// below), else 4 independent pairs.  The score
// tile S^T = K Q^T is one v_mfma_f32_16x16x32 per 16 keys x 16 queries at
// dh = 32 (plus one 16x16x16 for the last 16 features at dh = 48), with K as
// the MFMA "A" operand so each lane holds 4 keys of ONE query: the softmax
// max / sum are 2 in-lane steps + 2 cross-lane butterflies (lane ^ 16,
// lane ^ 32), all in fp32.  The normalised probabilities, rounded to the
// 16-bit type, are then directly the "B" operand of the P.V MFMA
// (v_mfma_f32_16x16x16, K = 16 keys); V is staged through LDS once per wave
// because that product needs it key-contiguous per lane.  Each lane ends with
// 4 consecutive output features of one query row: 8-byte stores.
// Q, K, V are read straight out of the packed projection through strides.
//
// fp32 path: one thread per (env, head, query), two passes over the keys
// (parity configuration only).
//
// Semantics: softmax_k(q.k / sqrt(dh) + bias_k) v with the additive key bias
// 0 / -2^14 of the reference (python/policy.py:686-690, :1257-1260); masked
// keys get exactly zero weight, which the kernel realises by skipping them.
// Replaces python/beat_arena_env/csrc/small_attn.cu:228-332 (attn29_fwd) and
// the SDPA fallbacks of python/fp16_linear.py:866-909.
#include "bsrl_common.h"

namespace {

struct AttnArgs {
    const void *q, *k, *v;
    int64_t q_bs, q_rs, k_bs, k_rs, v_bs, v_rs;
    const void* key_bias;      // (B, T) in dtype, or NULL
    const int32_t* n_valid;    // (B,), or NULL
    void* out;
    int64_t B; int T, TQ, H;
    float scale;
};

constexpr int kMaxKT = 3;      // key tiles of 16 (T <= 48)

template <typename DT, int DH>
__global__ __launch_bounds__(256) void attn_mfma_kernel(AttnArgs a) {
    constexpr int VLD = DH + 8;                 // LDS row pitch (halves): 16-byte aligned, bank-spread
    constexpr int FT = DH / 16;                 // output feature tiles
    __shared__ __attribute__((aligned(16))) u16 vs[4][kMaxKT * 16 * VLD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t pair = (int64_t)blockIdx.x * 4 + wave;
    const bool live = pair < a.B * a.H;
    const int64_t b = live ? pair / a.H : 0;
    const int h = live ? (int)(pair % a.H) : 0;
    const int T = a.T, TQ = a.TQ;
    const int nkt = (T + 15) >> 4, nqt = (TQ + 15) >> 4;
    const u16* qp = static_cast<const u16*>(a.q) + b * a.q_bs + h * DH;
    const u16* kp = static_cast<const u16*>(a.k) + b * a.k_bs + h * DH;
    const u16* vp = static_cast<const u16*>(a.v) + b * a.v_bs + h * DH;
    u16* myv = vs[wave];

    // V rows -> LDS (zero rows beyond T: their probabilities are 0, but 0 * junk must stay 0); every load is
    // issued before the first LDS write, so the staging costs one memory round trip, not one per piece
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int VPR = DH / 8, VNIT = (kMaxKT * 16 * VPR + WAVE - 1) / WAVE;
    u32x4 vbuf[VNIT];
#pragma unroll
    for (int it = 0; it < VNIT; ++it) {
        const int c = it * WAVE + lane, row = c / VPR, part = c % VPR;
        vbuf[it] = (u32x4){0u, 0u, 0u, 0u};
        if (row < T) vbuf[it] = *reinterpret_cast<const u32x4*>(vp + (int64_t)row * a.v_rs + part * 8);
    }
#pragma unroll
    for (int it = 0; it < VNIT; ++it) {
        const int c = it * WAVE + lane, row = c / VPR, part = c % VPR;
        if (row < nkt * 16) *reinterpret_cast<u32x4*>(myv + row * VLD + part * 8) = vbuf[it];
    }
    // K fragments (A operand): lane (key = r16, k-block g)
    s16x8 kf[kMaxKT]; s16x4 kf2[kMaxKT];
#pragma unroll
    for (int kt = 0; kt < kMaxKT; ++kt) {
        int key = kt * 16 + r16; key = key < T ? key : T - 1;
        const u16* p = kp + (int64_t)key * a.k_rs;
        kf[kt] = (s16x8){0, 0, 0, 0, 0, 0, 0, 0}; kf2[kt] = (s16x4){0, 0, 0, 0};
        if (kt < nkt) {
            kf[kt] = *reinterpret_cast<const s16x8*>(p + g * 8);
            if (DH == 48) kf2[kt] = *reinterpret_cast<const s16x4*>(p + 32 + g * 4);
        }
    }
    // per-lane key validity / additive bias for keys 16*kt + 4*g + i
    float kb[kMaxKT][4];
    const int nv = a.n_valid ? a.n_valid[b] : T;
#pragma unroll
    for (int kt = 0; kt < kMaxKT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kt * 16 + g * 4 + i;
            float bias = 0.f;
            if (key >= T || key > nv) bias = -INFINITY;
            else if (a.key_bias) {
                const float kbv = DT::to_f(static_cast<const u16*>(a.key_bias)[b * T + key]);
                bias = kbv < -0.5f * BSRL_MASK_BIAS ? -INFINITY : kbv;
            }
            kb[kt][i] = bias;
        }
    __syncthreads();
    // V^T fragments (A operand of P.V): lane (feature = r16, keys 4g..4g+3)
    s16x4 vf[kMaxKT][FT];
#pragma unroll
    for (int kt = 0; kt < kMaxKT; ++kt)
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
            vf[kt][ft] = (s16x4){0, 0, 0, 0};
            if (kt < nkt) {
#pragma unroll
                for (int i = 0; i < 4; ++i) vf[kt][ft][i] = (short)myv[(kt * 16 + g * 4 + i) * VLD + ft * 16 + r16];
            }
        }

    u16* op = static_cast<u16*>(a.out) + (b * TQ) * (int64_t)(a.H * DH) + h * DH;
    for (int qt = 0; qt < nqt; ++qt) {
        int qrow = qt * 16 + r16;
        const bool qlive = live && qrow < TQ;
        qrow = qrow < TQ ? qrow : TQ - 1;
        const u16* p = qp + (int64_t)qrow * a.q_rs;
        const s16x8 qf = *reinterpret_cast<const s16x8*>(p + g * 8);
        s16x4 qf2 = {0, 0, 0, 0};
        if (DH == 48) qf2 = *reinterpret_cast<const s16x4*>(p + 32 + g * 4);
        float s[kMaxKT][4];
        float m = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < kMaxKT; ++kt) {
            // The K = 32 and K = 16 products go to SEPARATE accumulators and are summed on the
            // VALU: chaining a 16x16x16 MFMA onto the accumulator of a 16x16x32 one lost the
            // first product on gfx950 (measured), same-shape chains are fine.
            f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
            if (kt < nkt) {
                acc = DT::mfma32(kf[kt], qf, acc);
                if (DH == 48) acc2 = DT::mfma16(kf2[kt], qf2, acc2);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[kt][i] = (acc[i] + acc2[i]) * a.scale + kb[kt][i];
                m = fmaxf(m, s[kt][i]);
            }
        }
        m = fmaxf(m, __shfl_xor(m, 16, WAVE));
        m = fmaxf(m, __shfl_xor(m, 32, WAVE));
        float sum = 0.f;
#pragma unroll
        for (int kt = 0; kt < kMaxKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) { s[kt][i] = __expf(s[kt][i] - m); sum += s[kt][i]; }
        sum += __shfl_xor(sum, 16, WAVE);
        sum += __shfl_xor(sum, 32, WAVE);
        const float inv = 1.0f / sum;
        s16x4 pf[kMaxKT];
#pragma unroll
        for (int kt = 0; kt < kMaxKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) pf[kt][i] = (short)DT::from_f(s[kt][i] * inv);
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
            f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kt = 0; kt < kMaxKT; ++kt) if (kt < nkt) o = DT::mfma16(vf[kt][ft], pf[kt], o);
            if (qlive) {
                uint2 ov;
                ov.x = DT::pack2(o[0], o[1]);
                ov.y = DT::pack2(o[2], o[3]);
                *reinterpret_cast<uint2*>(op + (int64_t)qrow * (a.H * DH) + ft * 16 + g * 4) = ov;
            }
        }
    }
}

// ---- one workgroup per env ---------------------------------------------------------------------------------------
// The H heads of ONE env in a workgroup (wave = head), T <= 32, H <= 8: the env's q, k, v rows come in and the output
// leaves as whole d-wide rows (consecutive threads on consecutive 16-byte pieces) through per-head LDS tiles, the
// workgroup is persistent and holds the next env's rows in registers while it computes.  The kernel above reads each
// head's dh-wide slices per wave - 16 rows x 64 / 96 B per instruction - and writes 8-byte pieces from the accumulator
// layout: 207 us at B = 16384, T = 29, 4 x 48 against ~150 us of traffic at the rate a copy reaches.  Same arithmetic,
// operation for operation.
typedef short s16x4t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ s16x4 tr16_rows(const u16* tile, int pitch, int k0, int c0, int lane) {
    // 16x16x16 operand whose contraction index runs over the rows of a row-major LDS tile: lane (i, g) ends with rows
    // k0 + 4 g + {0..3} of column c0 + i (lanes 4 r + s of a 16-lane group present row k0 + 4 g + r, columns c0 + 4 s ..)
    const int i = lane & 15, g = lane >> 4;
    const u16* p = tile + (k0 + 4 * g + (i >> 2)) * pitch + c0 + 4 * (i & 3);
    typedef __attribute__((address_space(3))) s16x4t* lptr;
    const s16x4t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p));
    return (s16x4){t[0], t[1], t[2], t[3]};
}

template <typename DT, int DH>
__global__ __launch_bounds__(512) void attn_mfma_coop_kernel(AttnArgs a, int wave_elems) {
    constexpr int DHP = DH + 8;                 // LDS row pitch (elements): 8 consecutive rows on 8 different 16-byte slots
    constexpr int FT = DH / 16, NKT = 2;
    constexpr int PPR = DH / 8, NIT = (NKT * 16 * PPR + WAVE - 1) / WAVE;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) u16 smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int T = a.T, TQ = a.TQ, H = a.H;
    const int nkt = (T + 15) >> 4, nqt = (TQ + 15) >> 4;
    const int TP = nkt * 16, TQP = nqt * 16;
    u16* Qs = smem + (int64_t)wave * wave_elems;
    u16* Ks = Qs + TQP * DHP;
    u16* Vs = Ks + TP * DHP;
    const int offs[3] = {0, TQP * DHP, TQP * DHP + TP * DHP};
    const int nrows[3] = {TQ, T, T}, prows[3] = {TQP, TP, TP};
    const int64_t rss[3] = {a.q_rs, a.k_rs, a.v_rs};
    // piece c = it * blockDim + tid of a matrix is (row c / rp, head (c % rp) / PPR, part (c % rp) % PPR)
    const int rp = H * PPR, nthr = (int)blockDim.x, tid = (int)threadIdx.x;
    const int row_step = nthr / rp, cp_step = nthr % rp, row_first = tid / rp, cp_first = tid % rp;
    u32x4 buf[3][NIT];
    u16 kraw[NKT][4];
    int nv_next = 0;
    auto fetch = [&](int64_t be) __attribute__((always_inline)) {
        const u16* srcs[3] = {static_cast<const u16*>(a.q) + be * a.q_bs, static_cast<const u16*>(a.k) + be * a.k_bs,
                              static_cast<const u16*>(a.v) + be * a.v_bs};
#pragma unroll
        for (int mtx = 0; mtx < 3; ++mtx) {
            int row = row_first, cp = cp_first;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                buf[mtx][it] = (u32x4){0u, 0u, 0u, 0u};
                if (row < nrows[mtx]) buf[mtx][it] = *reinterpret_cast<const u32x4*>(srcs[mtx] + (int64_t)row * rss[mtx] + (cp / PPR) * DH + (cp % PPR) * 8);
                row += row_step; cp += cp_step;
                if (cp >= rp) { cp -= rp; ++row; }
            }
        }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kt * 16 + g * 4 + i;
                kraw[kt][i] = 0;
                if (a.key_bias && key < T) kraw[kt][i] = static_cast<const u16*>(a.key_bias)[be * T + key];
            }
        nv_next = a.n_valid ? a.n_valid[be] : T;
    };
    int64_t b = blockIdx.x;
    fetch(b);
    for (;;) {
#pragma unroll
        for (int mtx = 0; mtx < 3; ++mtx) {
            int row = row_first, cp = cp_first;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                if (row < prows[mtx]) *reinterpret_cast<u32x4*>(smem + (int64_t)(cp / PPR) * wave_elems + offs[mtx] + row * DHP + (cp % PPR) * 8) = buf[mtx][it];
                row += row_step; cp += cp_step;
                if (cp >= rp) { cp -= rp; ++row; }
            }
        }
        float kb[NKT][4];
        const int nv = nv_next;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kt * 16 + g * 4 + i;
                float bias = 0.f;
                if (key >= T || key > nv) bias = -INFINITY;
                else if (a.key_bias) {
                    const float kbv = DT::to_f(kraw[kt][i]);
                    bias = kbv < -0.5f * BSRL_MASK_BIAS ? -INFINITY : kbv;
                }
                kb[kt][i] = bias;
            }
        __syncthreads();
        const int64_t b_next = b + gridDim.x;
        const bool more = b_next < a.B;
        if (more) fetch(b_next);                   // in flight during this env's arithmetic

        // K fragments (A operand): lane (key = r16, k-block g); V^T fragments (A operand of P.V): lane (feature r16, keys 4g..)
        s16x8 kf[NKT]; s16x4 kf2[NKT]; s16x4 vf[NKT][FT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            kf[kt] = (s16x8){0, 0, 0, 0, 0, 0, 0, 0}; kf2[kt] = (s16x4){0, 0, 0, 0};
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) vf[kt][ft] = (s16x4){0, 0, 0, 0};
            if (kt < nkt) {
                const u16* p = Ks + (kt * 16 + r16) * DHP;
                kf[kt] = *reinterpret_cast<const s16x8*>(p + g * 8);
                if (DH == 48) kf2[kt] = *reinterpret_cast<const s16x4*>(p + 32 + g * 4);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) vf[kt][ft] = tr16_rows(Vs, DHP, kt * 16, ft * 16, lane);
            }
        }
        for (int qt = 0; qt < nqt; ++qt) {
            u16* qrowp = Qs + (qt * 16 + r16) * DHP;
            const s16x8 qf = *reinterpret_cast<const s16x8*>(qrowp + g * 8);
            s16x4 qf2 = {0, 0, 0, 0};
            if (DH == 48) qf2 = *reinterpret_cast<const s16x4*>(qrowp + 32 + g * 4);
            float s[NKT][4];
            float m = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};       // separate accumulators, as above
                if (kt < nkt) {
                    acc = DT::mfma32(kf[kt], qf, acc);
                    if (DH == 48) acc2 = DT::mfma16(kf2[kt], qf2, acc2);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[kt][i] = (acc[i] + acc2[i]) * a.scale + kb[kt][i];
                    m = fmaxf(m, s[kt][i]);
                }
            }
            m = fmaxf(m, __shfl_xor(m, 16, WAVE));
            m = fmaxf(m, __shfl_xor(m, 32, WAVE));
            float sum = 0.f;
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) { s[kt][i] = __expf(s[kt][i] - m); sum += s[kt][i]; }
            sum += __shfl_xor(sum, 16, WAVE);
            sum += __shfl_xor(sum, 32, WAVE);
            const float inv = 1.0f / sum;
            s16x4 pf[NKT];
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[kt][i] = (short)DT::from_f(s[kt][i] * inv);
            uint2 ov[FT];
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kt = 0; kt < NKT; ++kt) if (kt < nkt) o = DT::mfma16(vf[kt][ft], pf[kt], o);
                ov[ft].x = DT::pack2(o[0], o[1]);
                ov[ft].y = DT::pack2(o[2], o[3]);
            }
            // the query rows of this tile are in registers: the output takes their place until the rows leave
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) *reinterpret_cast<uint2*>(qrowp + ft * 16 + g * 4) = ov[ft];
        }
        __syncthreads();
        {
            u16* op = static_cast<u16*>(a.out) + (b * TQ) * (int64_t)(H * DH);
            int row = row_first, cp = cp_first;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                if (row < TQ)
                    *reinterpret_cast<u32x4*>(op + (int64_t)row * (H * DH) + (cp / PPR) * DH + (cp % PPR) * 8) =
                        *reinterpret_cast<const u32x4*>(smem + (int64_t)(cp / PPR) * wave_elems + row * DHP + (cp % PPR) * 8);
                row += row_step; cp += cp_step;
                if (cp >= rp) { cp -= rp; ++row; }
            }
        }
        if (!more) break;
        __syncthreads();                           // every thread is done reading the output tiles
        b = b_next;
    }
}

__global__ __launch_bounds__(256) void attn_f32_kernel(AttnArgs a, int dh) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = a.B * a.H * a.TQ;
    if (idx >= total) return;
    const int qi = (int)(idx % a.TQ);
    const int h = (int)((idx / a.TQ) % a.H);
    const int64_t b = idx / ((int64_t)a.TQ * a.H);
    const float* qp = static_cast<const float*>(a.q) + b * a.q_bs + (int64_t)qi * a.q_rs + h * dh;
    const float* kp = static_cast<const float*>(a.k) + b * a.k_bs + h * dh;
    const float* vp = static_cast<const float*>(a.v) + b * a.v_bs + h * dh;
    const float* kbp = a.key_bias ? static_cast<const float*>(a.key_bias) + b * a.T : nullptr;
    const int nv = a.n_valid ? a.n_valid[b] : a.T;
    float q[64], acc[64];
#pragma unroll
    for (int f = 0; f < 64; ++f) { q[f] = f < dh ? qp[f] : 0.f; acc[f] = 0.f; }
    float m = -INFINITY;
    for (int key = 0; key < a.T; ++key) {
        if (key > nv) continue;
        float s = 0.f;
#pragma unroll
        for (int f = 0; f < 64; ++f) if (f < dh) s = fmaf(q[f], kp[(int64_t)key * a.k_rs + f], s);
        s = s * a.scale + (kbp ? kbp[key] : 0.f);
        m = fmaxf(m, s);
    }
    float sum = 0.f;
    for (int key = 0; key < a.T; ++key) {
        if (key > nv) continue;
        float s = 0.f;
#pragma unroll
        for (int f = 0; f < 64; ++f) if (f < dh) s = fmaf(q[f], kp[(int64_t)key * a.k_rs + f], s);
        s = s * a.scale + (kbp ? kbp[key] : 0.f);
        const float e = expf(s - m);
        sum += e;
#pragma unroll
        for (int f = 0; f < 64; ++f) if (f < dh) acc[f] = fmaf(e, vp[(int64_t)key * a.v_rs + f], acc[f]);
    }
    float* op = static_cast<float*>(a.out) + (b * a.TQ + qi) * (int64_t)(a.H * dh) + h * dh;
    const float inv = 1.0f / sum;
#pragma unroll
    for (int f = 0; f < 64; ++f) if (f < dh) op[f] = acc[f] * inv;
}

}  // namespace

extern "C" int bsrl_attn_fwd(const void* q, int64_t q_bs, int64_t q_rs, const void* k, int64_t k_bs, int64_t k_rs,
                             const void* v, int64_t v_bs, int64_t v_rs, const void* key_bias,
                             const int32_t* n_valid, void* out, int64_t B, int64_t T, int64_t TQ, int64_t H,
                             int64_t dh, int dtype, bsrl_stream stream) {
    if (!q || !k || !v || !out) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_fwd: null pointer");
    if (B < 0 || T <= 0 || TQ <= 0 || TQ > T || H <= 0 || dh <= 0)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_fwd: bad shape B=%lld T=%lld TQ=%lld H=%lld dh=%lld", (long long)B,
                  (long long)T, (long long)TQ, (long long)H, (long long)dh);
    if (key_bias && n_valid) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_fwd: pass key_bias or n_valid, not both");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_fwd: bad dtype");
    if (B == 0) return BSRL_OK;
    if (T > BSRL_MAX_T) return BSRL_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    AttnArgs a{q, k, v, q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, key_bias, n_valid, out, B, (int)T, (int)TQ, (int)H,
               (float)(1.0 / sqrt((double)dh))};
    if (dtype == BSRL_F32) {
        if (dh > 64) return BSRL_UNSUPPORTED;
        const int64_t total = B * H * TQ;
        hipLaunchKernelGGL(attn_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, a, (int)dh);
    } else {
        if (dh != 32 && dh != 48) return BSRL_UNSUPPORTED;
        const bool ok = bsrl_aligned(q, 16) && bsrl_aligned(k, 16) && bsrl_aligned(v, 16) && bsrl_aligned(out, 8) &&
                        q_bs % 8 == 0 && q_rs % 8 == 0 && k_bs % 8 == 0 && k_rs % 8 == 0 && v_bs % 8 == 0 && v_rs % 8 == 0;
        if (!ok) return BSRL_UNSUPPORTED;
        // one persistent workgroup per env (wave = head) where the shape allows
        const int tp = (int)((T + 15) / 16) * 16, tqp = (int)((TQ + 15) / 16) * 16;
        const int wave_elems = (tqp + 2 * tp) * ((int)dh + 8);
        const size_t lds = (size_t)H * wave_elems * sizeof(u16);
        if (H <= 8 && T <= 32 && lds <= 64 * 1024 && bsrl_aligned(out, 16) && (H * dh) % 8 == 0) {
            int cus = 256, dev = 0;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
            const int64_t resident = (int64_t)cus * (lds <= 40 * 1024 ? 4 : lds <= 53 * 1024 ? 3 : 2);
            const dim3 cgrid((unsigned)(B < resident ? B : resident)), cblock((unsigned)(64 * H));
            if (dtype == BSRL_F16) {
                if (dh == 32) hipLaunchKernelGGL((attn_mfma_coop_kernel<F16, 32>), cgrid, cblock, lds, st, a, wave_elems);
                else hipLaunchKernelGGL((attn_mfma_coop_kernel<F16, 48>), cgrid, cblock, lds, st, a, wave_elems);
            } else {
                if (dh == 32) hipLaunchKernelGGL((attn_mfma_coop_kernel<BF16, 32>), cgrid, cblock, lds, st, a, wave_elems);
                else hipLaunchKernelGGL((attn_mfma_coop_kernel<BF16, 48>), cgrid, cblock, lds, st, a, wave_elems);
            }
            BSRL_CHECK_LAUNCH("bsrl_attn_fwd");
            return BSRL_OK;
        }
        const unsigned grid = (unsigned)((B * H + 3) / 4);
        if (dtype == BSRL_F16) {
            if (dh == 32) hipLaunchKernelGGL((attn_mfma_kernel<F16, 32>), dim3(grid), dim3(256), 0, st, a);
            else hipLaunchKernelGGL((attn_mfma_kernel<F16, 48>), dim3(grid), dim3(256), 0, st, a);
        } else {
            if (dh == 32) hipLaunchKernelGGL((attn_mfma_kernel<BF16, 32>), dim3(grid), dim3(256), 0, st, a);
            else hipLaunchKernelGGL((attn_mfma_kernel<BF16, 48>), dim3(grid), dim3(256), 0, st, a);
        }
    }
    BSRL_CHECK_LAUNCH("bsrl_attn_fwd");
    return BSRL_OK;
}
