// Backward of the short-sequence masked multi-head attention (T <= 48 keys) for gfx950.
//
// Replaces fp16_gemm.attn29_bwd(q, k, v, bias, dout, dq, dk, dv) (reference
// python/beat_arena_env/csrc/small_attn.cu:345-463, 539-571; callers python/fp16_linear.py:930-1000):
// the probabilities are recomputed from q, k and the key mask exactly as the forward computes them
// (fp32 scores, fp32 softmax), then
//     dP = dO V^T,  dS = P * (dP - rowsum(P * dP)),  dQ = scale dS K,  dK = scale dS^T Q,  dV = P^T dO
// and the three gradients are written through strides, so they may be column slices of one packed
// q|k|v gradient buffer (what the reference's callers pass).
//
// 16-bit path: one wave64 per (env, head); a workgroup is the H heads of one env where they fit (persistent, the next
// env's rows prefetched in registers), else 2 independent pairs.  q, k, v, dO are
// staged once in LDS as they lie in memory (rows = tokens); every product is a chain of
// v_mfma_f32_16x16x16 with the operand orientation each one needs:
//   S^T = K Q^T and dP^T = V dO^T contract over features: both operands are plain 8-byte row reads;
//   a lane ends with 4 consecutive KEYS of one query, so the softmax and the rowsum are in-lane
//   steps plus two butterflies (lane ^ 16, lane ^ 32), and dS^T packs straight into the B operand of
//   dQ^T = K^T dS^T, whose A operand (K^T) is an LDS transpose load (ds_read_b64_tr_b16);
//   dV^T = dO^T P and dK^T = Q^T dS contract over QUERIES: P and dS of the current 16-query tile go
//   through a 16-row LDS tile and both operands come back through transpose loads.
// Every output lane holds 4 consecutive features of one token; the gradients take the place of q, k, v in LDS and
// leave as 16-byte pieces of whole rows.  dK^T / dV^T stay in accumulators across the query tiles.  HBM traffic:
// q, k, v, dO read once, dq, dk, dv written once.  B = 16384, T = 29, 4 x 48: 454 us with per-wave slices and 8-byte
// stores, 417 us with whole rows per workgroup, 319 us (4.0 TB/s) with the persistent prefetching form.
//
// fp32 path (parity configuration): one wave per (env, head) on LDS-staged fp32 tiles, plain FMA loops.
#include "bsrl_common.h"

namespace {

struct AttnBwdArgs {
    const void *q, *k, *v, *dout;
    int64_t q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, do_bs, do_rs;
    const void* key_bias; const int32_t* n_valid;
    void *dq, *dk, *dv;
    int64_t dq_bs, dq_rs, dk_bs, dk_rs, dv_bs, dv_rs;
    int64_t B; int T, TQ, H;
    float scale;
    int wave_elems;            // 16-bit path: LDS elements per wave
    int out16;                 // 16-bit path: gradient rows may leave as 16-byte pieces (else 8-byte)
};

typedef short s16x4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));

// 16x16x16 operand whose contraction index runs over the ROWS of a row-major LDS tile: lane (i = lane % 16,
// g = lane / 16) ends with rows k0 + 4 g + {0..3} of column c0 + i.  Lanes 4 r + s of a 16-lane group present
// the 4 elements at column c0 + 4 s of row k0 + 4 g + r; the hardware hands lane i element i of rows 0..3.
__device__ __forceinline__ s16x4 tr16(const u16* tile, int pitch, int k0, int c0, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const u16* p = tile + (k0 + 4 * g + (i >> 2)) * pitch + c0 + 4 * (i & 3);
    typedef __attribute__((address_space(3))) s16x4v* lptr;
    const s16x4v t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p));
    return (s16x4){t[0], t[1], t[2], t[3]};
}
// operand whose contraction index runs ALONG a row: lane (i, g) reads columns c0 + 4 g .. + 3 of row r0 + i
__device__ __forceinline__ s16x4 row16(const u16* tile, int pitch, int r0, int c0, int lane) {
    return *reinterpret_cast<const s16x4*>(tile + (r0 + (lane & 15)) * pitch + c0 + 4 * (lane >> 4));
}

// COOP: a workgroup is the H heads of ONE env (wave = head) and moves the env's rows together: q, k, v, dO come in and
// dq, dk, dv leave as whole d-wide rows (consecutive threads on consecutive 16-byte pieces), through the per-head LDS
// tiles.  Otherwise (H > 8, or H heads do not fit the LDS) a workgroup is 2 independent (env, head) pairs and every wave
// moves its own dh-wide slices.  Written straight from the accumulators (a lane holds 4 consecutive features of one
// token) the gradients left as 32-byte pieces and the stores cost 130 us of a 450 us kernel at B = 16384, T = 29, 4 x 48.
// NKT: key tiles of 16 the instantiation is sized for (2 for T <= 32: 60 fewer registers than 3, which is what lets the
// persistent form keep the next env's rows in registers without spilling)
template <typename DT, int DH, bool COOP, int NKT>
__global__ __launch_bounds__(COOP ? 512 : 128) void attn_bwd_mfma_kernel(AttnBwdArgs a) {
    constexpr int DHP = DH == 32 ? 48 : 56;     // LDS row pitch of the token tiles (elements)
    constexpr int FT = DH / 16;
    extern __shared__ __attribute__((aligned(16))) u16 smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    int64_t b; int h;
    if (COOP) { b = blockIdx.x; h = wave; }
    else {
        const int64_t pair = (int64_t)blockIdx.x * 2 + wave;
        if (pair >= a.B * a.H) return;                               // waves are independent: no workgroup barrier in this mode
        b = pair / a.H;
        h = (int)(pair % a.H);
    }
    // the group that moves rows together: all threads and all heads of the workgroup (COOP) or this wave and its head
    const int gh = COOP ? a.H : 1, h0 = COOP ? 0 : h;
    const int gthreads = COOP ? (int)blockDim.x : WAVE, gt = COOP ? (int)threadIdx.x : lane;
    const int T = a.T, TQ = a.TQ;
    const int nkt = (T + 15) >> 4, nqt = (TQ + 15) >> 4;
    const int TP = nkt * 16, TQP = nqt * 16, PP = TP + 8;
    u16* Qs = smem + (int64_t)wave * a.wave_elems;
    u16* dOs = Qs + TQP * DHP;
    u16* Ks = dOs + TQP * DHP;
    u16* Vs = Ks + TP * DHP;
    u16* Ps = Vs + TP * DHP;
    u16* dSs = Ps + 16 * PP;

    // stage the pair's q, dO (TQ rows) and k, v (T rows), zero rows up to the tile edge.  All global loads are
    // issued before the first LDS write: one memory round trip for the four matrices instead of one per piece.
    constexpr int PPR = DH / 8;                                     // 16-byte pieces per row
    constexpr int NIT = (NKT * 16 * PPR + WAVE - 1) / WAVE;      // pieces per lane and matrix, at most
    u32x4v buf[4][NIT];                                             // native vectors: arrays of the uint4 class that live across a loop stay in scratch
    u16 kraw[NKT][4];                                            // key bias of keys 16 kt + 4 g + e, raw
    int nv_next = 0;
    const int64_t rss[4] = {a.q_rs, a.do_rs, a.k_rs, a.v_rs};
    const int nrows[4] = {TQ, TQ, T, T}, prows[4] = {TQP, TQP, TP, TP};
    const int offs[4] = {0, TQP * DHP, 2 * TQP * DHP, 2 * TQP * DHP + TP * DHP};          // Qs, dOs, Ks, Vs inside a wave's region
    // piece c = it * gthreads + gt of a matrix is (row c / rp, head (c % rp) / PPR, part (c % rp) % PPR)
    const int rp = gh * PPR;
    const int row_step = gthreads / rp, cp_step = gthreads % rp;
    const int row_first = gt / rp, cp_first = gt % rp;
    auto tile_of = [&](int hh) __attribute__((always_inline)) { return smem + (int64_t)(COOP ? hh : wave) * a.wave_elems; };
    // all global loads of an env (the four matrices, the key bias, the valid count) are issued together
    auto fetch = [&](int64_t be) __attribute__((always_inline)) {
        const u16* srcs[4] = {static_cast<const u16*>(a.q) + be * a.q_bs + h0 * DH, static_cast<const u16*>(a.dout) + be * a.do_bs + h0 * DH,
                              static_cast<const u16*>(a.k) + be * a.k_bs + h0 * DH, static_cast<const u16*>(a.v) + be * a.v_bs + h0 * DH};
#pragma unroll
        for (int mtx = 0; mtx < 4; ++mtx) {
            int row = row_first, cp = cp_first;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                buf[mtx][it] = (u32x4v){0u, 0u, 0u, 0u};
                if (row < nrows[mtx]) buf[mtx][it] = *reinterpret_cast<const u32x4v*>(srcs[mtx] + (int64_t)row * rss[mtx] + (cp / PPR) * DH + (cp % PPR) * 8);
                row += row_step; cp += cp_step;
                if (cp >= rp) { cp -= rp; ++row; }
            }
        }
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = kt * 16 + g * 4 + e;
                kraw[kt][e] = 0;
                if (a.key_bias && key < T) kraw[kt][e] = static_cast<const u16*>(a.key_bias)[be * T + key];
            }
        nv_next = a.n_valid ? a.n_valid[be] : T;
    };
    fetch(b);
  for (;;) {                                                        // COOP: a persistent workgroup walks envs b, b + grid, ...
#pragma unroll
    for (int mtx = 0; mtx < 4; ++mtx) {
        int row = row_first, cp = cp_first;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            if (row < prows[mtx]) *reinterpret_cast<u32x4v*>(tile_of(cp / PPR) + offs[mtx] + row * DHP + (cp % PPR) * 8) = buf[mtx][it];
            row += row_step; cp += cp_step;
            if (cp >= rp) { cp -= rp; ++row; }
        }
    }
    // additive bias / validity of keys 16 kt + 4 g + e, as the forward applies them
    float kb[NKT][4];
    const int nv = nv_next;
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int key = kt * 16 + g * 4 + e;
            float bias = 0.f;
            if (key >= T || key > nv) bias = -INFINITY;
            else if (a.key_bias) {
                const float kbv = DT::to_f(kraw[kt][e]);
                bias = kbv < -0.5f * BSRL_MASK_BIAS ? -INFINITY : kbv;
            }
            kb[kt][e] = bias;
        }
    if (COOP) __syncthreads();
    // the next env's loads fly during this env's arithmetic (their registers are free until the next tile fill)
    const int64_t b_next = b + gridDim.x;
    const bool more = COOP && b_next < a.B;
    if (more) fetch(b_next);

    f32x4 dkt[FT][NKT], dvt[FT][NKT];      // dK^T, dV^T: lane holds features 16 ft + 4 g + e of key 16 kt + r16
#pragma unroll
    for (int ft = 0; ft < FT; ++ft)
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) { dkt[ft][kt] = (f32x4){0.f, 0.f, 0.f, 0.f}; dvt[ft][kt] = (f32x4){0.f, 0.f, 0.f, 0.f}; }

    for (int qt = 0; qt < nqt; ++qt) {
        // S^T and dP^T tiles: lane holds keys 16 kt + 4 g + e of query 16 qt + r16
        float s[NKT][4], dp[NKT][4];
        float m = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            f32x4 sa = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
            if (kt < nkt) {
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    sa = DT::mfma16(row16(Ks, DHP, kt * 16, ft * 16, lane), row16(Qs, DHP, qt * 16, ft * 16, lane), sa);
                    da = DT::mfma16(row16(Vs, DHP, kt * 16, ft * 16, lane), row16(dOs, DHP, qt * 16, ft * 16, lane), da);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[kt][e] = sa[e] * a.scale + kb[kt][e];
                dp[kt][e] = da[e];
                m = fmaxf(m, s[kt][e]);
            }
        }
        m = fmaxf(m, __shfl_xor(m, 16, WAVE));
        m = fmaxf(m, __shfl_xor(m, 32, WAVE));
        float sum = 0.f;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) { s[kt][e] = __expf(s[kt][e] - m); sum += s[kt][e]; }
        sum += __shfl_xor(sum, 16, WAVE);
        sum += __shfl_xor(sum, 32, WAVE);
        const float inv = 1.0f / sum;
        float dsum = 0.f;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) { s[kt][e] *= inv; dsum += s[kt][e] * dp[kt][e]; }      // s = P from here on
        dsum += __shfl_xor(dsum, 16, WAVE);
        dsum += __shfl_xor(dsum, 32, WAVE);
        s16x4 dsf[NKT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            uint32_t pw[2], dw[2];
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
                const float d0 = s[kt][e] * (dp[kt][e] - dsum), d1 = s[kt][e + 1] * (dp[kt][e + 1] - dsum);
                pw[e >> 1] = DT::pack2(s[kt][e], s[kt][e + 1]);
                dw[e >> 1] = DT::pack2(d0, d1);
            }
            dsf[kt] = __builtin_bit_cast(s16x4, make_uint2(dw[0], dw[1]));
            if (kt < nkt) {                     // row = the lane's query, 4 consecutive keys: one 8-byte LDS write each
                *reinterpret_cast<uint2*>(Ps + r16 * PP + kt * 16 + 4 * g) = make_uint2(pw[0], pw[1]);
                *reinterpret_cast<uint2*>(dSs + r16 * PP + kt * 16 + 4 * g) = make_uint2(dw[0], dw[1]);
            }
        }
        // dQ^T = K^T dS^T: A = K^T (transpose load, contraction over keys), B = dS^T from registers
        uint2 dqv[FT];
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) {
            f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kt = 0; kt < NKT; ++kt)
                if (kt < nkt) o = DT::mfma16(tr16(Ks, DHP, kt * 16, ft * 16, lane), dsf[kt], o);
            dqv[ft].x = DT::pack2(o[0] * a.scale, o[1] * a.scale);
            dqv[ft].y = DT::pack2(o[2] * a.scale, o[3] * a.scale);
        }
        // dV^T += dO^T P, dK^T += Q^T dS: contraction over this tile's 16 queries, both operands transposed
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            if (kt < nkt) {
                const s16x4 pb = tr16(Ps, PP, 0, kt * 16, lane), db = tr16(dSs, PP, 0, kt * 16, lane);
#pragma unroll
                for (int ft = 0; ft < FT; ++ft) {
                    dvt[ft][kt] = DT::mfma16(tr16(dOs, DHP, qt * 16, ft * 16, lane), pb, dvt[ft][kt]);
                    dkt[ft][kt] = DT::mfma16(tr16(Qs, DHP, qt * 16, ft * 16, lane), db, dkt[ft][kt]);
                }
            }
        }
        // this tile's q rows have had their last read: dQ takes their place until the rows leave
#pragma unroll
        for (int ft = 0; ft < FT; ++ft) *reinterpret_cast<uint2*>(Qs + (qt * 16 + r16) * DHP + ft * 16 + 4 * g) = dqv[ft];
    }
    // dK and dV take the place of k and v (every read of them is behind this wave), then the rows leave together
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
        if (kt < nkt) {
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                uint2 kv, vv;
                kv.x = DT::pack2(dkt[ft][kt][0] * a.scale, dkt[ft][kt][1] * a.scale);
                kv.y = DT::pack2(dkt[ft][kt][2] * a.scale, dkt[ft][kt][3] * a.scale);
                vv.x = DT::pack2(dvt[ft][kt][0], dvt[ft][kt][1]);
                vv.y = DT::pack2(dvt[ft][kt][2], dvt[ft][kt][3]);
                *reinterpret_cast<uint2*>(Ks + (kt * 16 + r16) * DHP + ft * 16 + 4 * g) = kv;
                *reinterpret_cast<uint2*>(Vs + (kt * 16 + r16) * DHP + ft * 16 + 4 * g) = vv;
            }
        }
    }
    if (COOP) __syncthreads();
    u16* outs[3] = {static_cast<u16*>(a.dq) + b * a.dq_bs + h0 * DH, static_cast<u16*>(a.dk) + b * a.dk_bs + h0 * DH,
                    static_cast<u16*>(a.dv) + b * a.dv_bs + h0 * DH};
    const int64_t ors[3] = {a.dq_rs, a.dk_rs, a.dv_rs};
    const int orows[3] = {TQ, T, T}, ooffs[3] = {offs[0], offs[2], offs[3]};
#pragma unroll
    for (int mtx = 0; mtx < 3; ++mtx) {
        int row = row_first, cp = cp_first;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            if (row < orows[mtx]) {
                const uint4 v = *reinterpret_cast<const uint4*>(tile_of(cp / PPR) + ooffs[mtx] + row * DHP + (cp % PPR) * 8);
                u16* dst = outs[mtx] + (int64_t)row * ors[mtx] + (cp / PPR) * DH + (cp % PPR) * 8;
                if (a.out16) *reinterpret_cast<uint4*>(dst) = v;
                else { *reinterpret_cast<uint2*>(dst) = make_uint2(v.x, v.y); *reinterpret_cast<uint2*>(dst + 4) = make_uint2(v.z, v.w); }
            }
            row += row_step; cp += cp_step;
            if (cp >= rp) { cp -= rp; ++row; }
        }
    }
    if (!more) break;
    __syncthreads();                               // every thread is done reading the gradient tiles
    b = b_next;
  }
}

// fp32: one wave per (env, head); tiles in LDS, thread-per-element loops.  dh <= 48, T <= 48.
__global__ __launch_bounds__(64) void attn_bwd_f32_kernel(AttnBwdArgs a, int dh) {
    __shared__ float Qs[48 * 49], Ks[48 * 49], Vs[48 * 49], Os[48 * 49], Pm[48 * 49], Dm[48 * 49];
    const int lane = threadIdx.x;
    const int64_t pair = blockIdx.x;
    const int64_t b = pair / a.H;
    const int h = (int)(pair % a.H);
    const int T = a.T, TQ = a.TQ;
    const float* qp = static_cast<const float*>(a.q) + b * a.q_bs + h * dh;
    const float* kp = static_cast<const float*>(a.k) + b * a.k_bs + h * dh;
    const float* vp = static_cast<const float*>(a.v) + b * a.v_bs + h * dh;
    const float* op = static_cast<const float*>(a.dout) + b * a.do_bs + h * dh;
    for (int i = lane; i < TQ * dh; i += 64) { const int r = i / dh, c = i % dh; Qs[r * 49 + c] = qp[(int64_t)r * a.q_rs + c]; Os[r * 49 + c] = op[(int64_t)r * a.do_rs + c]; }
    for (int i = lane; i < T * dh; i += 64) { const int r = i / dh, c = i % dh; Ks[r * 49 + c] = kp[(int64_t)r * a.k_rs + c]; Vs[r * 49 + c] = vp[(int64_t)r * a.v_rs + c]; }
    __syncthreads();
    const float* kbp = a.key_bias ? static_cast<const float*>(a.key_bias) + b * T : nullptr;
    const int nv = a.n_valid ? a.n_valid[b] : T;
    // scores and dP, one (query, key) per thread step
    for (int i = lane; i < TQ * T; i += 64) {
        const int qi = i / T, key = i % T;
        float s = 0.f, d = 0.f;
        for (int c = 0; c < dh; ++c) { s = fmaf(Qs[qi * 49 + c], Ks[key * 49 + c], s); d = fmaf(Os[qi * 49 + c], Vs[key * 49 + c], d); }
        float bias = 0.f;
        if (key > nv) bias = -INFINITY;
        else if (kbp) bias = kbp[key] < -0.5f * BSRL_MASK_BIAS ? -INFINITY : kbp[key];
        Pm[qi * 49 + key] = s * a.scale + bias;
        Dm[qi * 49 + key] = d;
    }
    __syncthreads();
    // softmax and dS per query row
    for (int qi = lane; qi < TQ; qi += 64) {
        float m = -INFINITY;
        for (int key = 0; key < T; ++key) m = fmaxf(m, Pm[qi * 49 + key]);
        float sum = 0.f;
        for (int key = 0; key < T; ++key) { const float e = expf(Pm[qi * 49 + key] - m); Pm[qi * 49 + key] = e; sum += e; }
        const float inv = 1.0f / sum;
        float dsum = 0.f;
        for (int key = 0; key < T; ++key) { const float p = Pm[qi * 49 + key] * inv; Pm[qi * 49 + key] = p; dsum = fmaf(p, Dm[qi * 49 + key], dsum); }
        for (int key = 0; key < T; ++key) Dm[qi * 49 + key] = Pm[qi * 49 + key] * (Dm[qi * 49 + key] - dsum);
    }
    __syncthreads();
    float* dqp = static_cast<float*>(a.dq) + b * a.dq_bs + h * dh;
    float* dkp = static_cast<float*>(a.dk) + b * a.dk_bs + h * dh;
    float* dvp = static_cast<float*>(a.dv) + b * a.dv_bs + h * dh;
    for (int i = lane; i < TQ * dh; i += 64) {
        const int qi = i / dh, c = i % dh;
        float o = 0.f;
        for (int key = 0; key < T; ++key) o = fmaf(Dm[qi * 49 + key], Ks[key * 49 + c], o);
        dqp[(int64_t)qi * a.dq_rs + c] = o * a.scale;
    }
    for (int i = lane; i < T * dh; i += 64) {
        const int key = i / dh, c = i % dh;
        float ok = 0.f, ov = 0.f;
        for (int qi = 0; qi < TQ; ++qi) { ok = fmaf(Dm[qi * 49 + key], Qs[qi * 49 + c], ok); ov = fmaf(Pm[qi * 49 + key], Os[qi * 49 + c], ov); }
        dkp[(int64_t)key * a.dk_rs + c] = ok * a.scale;
        dvp[(int64_t)key * a.dv_rs + c] = ov;
    }
}

}  // namespace

extern "C" int bsrl_attn_bwd(const void* q, int64_t q_bs, int64_t q_rs, const void* k, int64_t k_bs, int64_t k_rs,
                             const void* v, int64_t v_bs, int64_t v_rs, const void* key_bias, const int32_t* n_valid,
                             const void* dout, int64_t do_bs, int64_t do_rs,
                             void* dq, int64_t dq_bs, int64_t dq_rs, void* dk, int64_t dk_bs, int64_t dk_rs,
                             void* dv, int64_t dv_bs, int64_t dv_rs,
                             int64_t B, int64_t T, int64_t TQ, int64_t H, int64_t dh, int dtype, bsrl_stream stream) {
    if (!q || !k || !v || !dout || !dq || !dk || !dv) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_bwd: null pointer");
    if (B < 0 || T <= 0 || TQ <= 0 || TQ > T || H <= 0 || dh <= 0)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_bwd: bad shape B=%lld T=%lld TQ=%lld H=%lld dh=%lld", (long long)B,
                  (long long)T, (long long)TQ, (long long)H, (long long)dh);
    if (key_bias && n_valid) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_bwd: pass key_bias or n_valid, not both");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_bwd: bad dtype %d", dtype);
    if (T > BSRL_MAX_T) return BSRL_UNSUPPORTED;
    if (B == 0) return BSRL_OK;
    if (B * H > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_attn_bwd: too many (env, head) pairs");
    const double scale = 1.0 / sqrt((double)dh);
    AttnBwdArgs a{q, k, v, dout, q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, do_bs, do_rs, key_bias, n_valid, dq, dk, dv,
                  dq_bs, dq_rs, dk_bs, dk_rs, dv_bs, dv_rs, B, (int)T, (int)TQ, (int)H, (float)scale, 0, 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == BSRL_F32) {
        if (dh > 48) return BSRL_UNSUPPORTED;
        hipLaunchKernelGGL(attn_bwd_f32_kernel, dim3((unsigned)(B * H)), dim3(64), 0, st, a, (int)dh);
    } else {
        if (dh != 32 && dh != 48) return BSRL_UNSUPPORTED;
        // 16-byte row reads and 8-byte gradient stores through the strides
        const int64_t in_s[] = {q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, do_bs, do_rs};
        for (int64_t s : in_s) if (s % 8 != 0) return BSRL_UNSUPPORTED;
        const int64_t out_s[] = {dq_bs, dq_rs, dk_bs, dk_rs, dv_bs, dv_rs};
        for (int64_t s : out_s) if (s % 4 != 0) return BSRL_UNSUPPORTED;
        if (!bsrl_aligned(q, 16) || !bsrl_aligned(k, 16) || !bsrl_aligned(v, 16) || !bsrl_aligned(dout, 16) ||
            !bsrl_aligned(dq, 8) || !bsrl_aligned(dk, 8) || !bsrl_aligned(dv, 8)) return BSRL_UNSUPPORTED;
        const int dhp = dh == 32 ? 48 : 56;
        const int tp = (int)((T + 15) / 16) * 16, tqp = (int)((TQ + 15) / 16) * 16;
        a.wave_elems = (2 * tqp + 2 * tp) * dhp + 2 * 16 * (tp + 8);
        a.wave_elems = (a.wave_elems + 7) & ~7;                          // keep each wave's region 16-byte aligned
        a.out16 = 1;
        for (int64_t s : out_s) if (s % 8 != 0) a.out16 = 0;
        if (!bsrl_aligned(dq, 16) || !bsrl_aligned(dk, 16) || !bsrl_aligned(dv, 16)) a.out16 = 0;
        // one workgroup per env (wave = head) when the H heads' tiles fit twice into a CU's LDS
        const size_t wave_bytes = (size_t)a.wave_elems * sizeof(u16);
        // (T <= 32: with three key tiles the prefetched rows no longer fit the register file)
        const bool coop = H <= 8 && T <= 32 && (size_t)H * wave_bytes <= 80 * 1024;
        const size_t lds = (coop ? (size_t)H : 2) * wave_bytes;
        // COOP workgroups are persistent (two resident per CU by LDS) and prefetch their next env
        int cus = 256, dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
        const int64_t resident = (int64_t)cus * 2;
        const dim3 grid(coop ? (unsigned)(B < resident ? B : resident) : (unsigned)((B * H + 1) / 2)), block(coop ? (unsigned)(64 * H) : 128u);
#define AB_COOP(DT, DH) do { \
            auto kern = attn_bwd_mfma_kernel<DT, DH, true, 2>; \
            if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
                (void)hipGetLastError(); return BSRL_UNSUPPORTED; } \
            hipLaunchKernelGGL(kern, grid, block, lds, st, a); } while (0)
#define AB_T(DT, DH) do { \
            if (coop) AB_COOP(DT, DH); \
            else if (T <= 32) hipLaunchKernelGGL((attn_bwd_mfma_kernel<DT, DH, false, 2>), grid, block, lds, st, a); \
            else hipLaunchKernelGGL((attn_bwd_mfma_kernel<DT, DH, false, 3>), grid, block, lds, st, a); } while (0)
        if (dtype == BSRL_F16) { if (dh == 32) AB_T(F16, 32); else AB_T(F16, 48); }
        else { if (dh == 32) AB_T(BF16, 32); else AB_T(BF16, 48); }
#undef AB_T
#undef AB_COOP
    }
    BSRL_CHECK_LAUNCH("bsrl_attn_bwd");
    return BSRL_OK;
}
