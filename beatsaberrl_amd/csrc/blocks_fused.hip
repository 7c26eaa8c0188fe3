// The transformer block stack of the policy in ONE persistent kernel for gfx950.
//
// Shape class: up to 32 tokens per env (NotePolicy: 29), d = 128 / 192 / 256 as 4 x 32, 4 x 48 or
// 8 x 32 heads, FFN width a multiple of 32, ReLU or GELU, fp16 or bf16 operands with fp32 accumulate.
// Replaces, for the block stack of NotePolicy._forward_stacked (python/policy.py:1262-1306),
// the per-block launch train of Block.forward (python/policy.py:524-715): LayerNorm, packed
// q|k|v projection, attention, output projection + residual, LayerNorm, FFN + residual,
// with the final block restricted to its first n_queries rows (the reference's n_queries
// path, python/policy.py:533-539: exact, masking is key-side only).
//
// Mapping.  One wave64 owns one 16-row MFMA tile of one env (rows 16*rt .. 16*rt + 15) and
// carries that tile's fp32 residual stream in registers through every block (d/16 feature
// tiles x 4 VGPRs).  An env is a wave pair; a workgroup of 8 waves owns 4 envs.  Everything
// row-local (LayerNorm, projections, FFN with the hidden kept in registers) is wave-local,
// with the activation always the MFMA operand whose free index is the token, so an output
// fragment (4 consecutive features per lane) packs straight into the next GEMM's operand;
// the k order this implies is baked into the weight image.  Only attention crosses the two
// row tiles: each wave parks its K and V^T fragments of the current head in LDS, and after
// the next stage barrier reads both tiles' fragments back (scores^T = K Q^T, 8 keys per
// lane for one query; softmax by in-lane + two cross-lane steps; P V as 16x16x32 MFMAs
// over the 32 keys).
//
// What bounds it: every weight fragment (1 KB) read from LDS feeds ONE MFMA of the reading wave,
// so a CU asks its LDS for 4 x 1 KB per 16 cycles = 256 B/clk against 128 B/clk delivered
// (measured): the stack runs at the LDS read rate, ~750 cycles per 12 KB stage.  Giving a wave both
// row tiles of an env halves that traffic but needs ~450 registers, i.e. one wave per SIMD; built
// and measured (3-slot ring, fragment reads prefetched across the barrier), it came out level at
// d = 128 and slower at d = 192 (register spills), each stage then waiting on the L2 latency of the
// weight stream (~1500 cycles) with no second wave to cover it.
//
// Weights stream from L2 through a 2-slot LDS ring in stages of 2 * (d/32) fragments
// (8 or 12 KB) shared by the 8 waves: loads issued three stages ahead into registers,
// written to LDS one stage ahead, one barrier per stage.  All fp32 vectors (biases,
// LayerNorm affine) of all blocks stay resident in LDS.  HBM traffic is the token stream in
// and the stream(s) out.
#include "bsrl_common.h"
#include <type_traits>

namespace {

struct BlkArgs {
    const uint2* frags; const float* vec;
    const u16* x_in; const u16* key_bias; u16* x_res; u16* x_out;
    int64_t B; int n_layers, F, T, n_queries, total_stages;
};

template <typename DT> __device__ __forceinline__ uint32_t bpack2(float a, float b) {
    return DT::pack2(a, b);
}
template <> __device__ __forceinline__ uint32_t bpack2<F16>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
template <> __device__ __forceinline__ uint32_t bpack2<BF16>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
union BFrag8 { s16x8 v; uint32_t w[4]; uint2 h[2]; uint4 u; };
union BFrag4 { s16x4 v; uint32_t w[2]; uint2 h; };

__device__ __forceinline__ void blk_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// compile-time loop: the body sees its index as a constant (the loop unroller gives up on the
// larger bodies, and register arrays indexed by the loop variable would then live in scratch)
template <int I, int N, typename Fn> __device__ __forceinline__ void static_for(Fn&& fn) {   // fn: an always_inline lambda
    if constexpr (I < N) { fn(std::integral_constant<int, I>{}); static_for<I + 1, N>(fn); }
}

template <int D> struct Geo {
    static constexpr int NT = D / 16, KC = D / 32, SF = 2 * KC;          // feature tiles, k chunks, fragments per stage
    // a stage is consumed in NB bursts of FB fragments (KB k chunks of both feature tiles): one burst of LDS
    // reads, then its MFMAs; bursts are sized to keep the fragment registers at 16-24 VGPRs
    static constexpr int NB = SF > 12 ? 4 : 2, FB = SF / NB, KB = KC / NB;
    static constexpr int STAGE_U2 = SF * 128;                             // uint2 per stage
    static constexpr int U2PT = STAGE_U2 / 512;                           // uint2 per thread per stage (2 or 3)
    __host__ __device__ static constexpr int layer_stages(int F) { return 3 * NT / 2 + NT / 2 + 2 * (F / 32); }
    // per-block fp32 vector region (floats)
    static constexpr int LN1G = 0, LN1B = D, BQ = 2 * D, BK = 3 * D, BV = 4 * D, BOUT = 5 * D, LN2G = 6 * D, LN2B = 7 * D, B1 = 8 * D;
    __host__ __device__ static constexpr int b2(int F) { return 8 * D + F; }
    __host__ __device__ static constexpr int lv_size(int F) { return 9 * D + F; }
};

// Weight-stage pipeline: stage s lives in ring slot s & 1; its global loads were issued three
// stage-steps earlier into the register set of the same parity.  The registers are plain named
// locals (an indexed array would live in scratch and force a wait right after each load).
#define BADVANCE_P(P, RA, RB, RC, RD) do { \
        blk_barrier();                                   /* stage s complete in slot P; slot 1-P free */ \
        ring[1 - (P)][tid] = RA; \
        ring[1 - (P)][tid + 512] = RB; \
        if (G::U2PT >= 3) ring[1 - (P)][tid + 1024] = RC; \
        if (G::U2PT == 4) ring[1 - (P)][tid + 1536] = RD; \
        const uint2* src_ = img + (int64_t)pnext * G::STAGE_U2 + tid; \
        RA = src_[0]; \
        RB = src_[512]; \
        if (G::U2PT >= 3) RC = src_[1024]; \
        if (G::U2PT == 4) RD = src_[1536]; \
        pnext = pnext + 1 == a.total_stages ? 0 : pnext + 1; \
    } while (0)
#define BADVANCE(par) do { if (par) BADVANCE_P(1, pr0a, pr0b, pr0c, pr0d); else BADVANCE_P(0, pr1a, pr1b, pr1c, pr1d); } while (0)
#define BWFRAG(par, f) (__builtin_bit_cast(s16x8, reinterpret_cast<const uint4*>(ring[par])[(f) * 64 + lane]))
// every fragment of the current stage -> registers in one burst of LDS reads (one wait instead of one per MFMA)
// one burst of a stage (FB fragments) -> registers in one run of LDS reads (one wait instead of one per MFMA).
// BLOAD_BURST: burst b of a two-tile stage, W[ntl * KB + ci] = k chunk b * KB + ci of tile ntl;
// BLOAD_RANGE: fragments [first, first + FB).
#define BLOAD_BURST(par, W, b) s16x8 W[G::FB]; _Pragma("unroll") for (int f_ = 0; f_ < G::FB; ++f_) W[f_] = BWFRAG(par, (b) * G::FB + f_)
#define BLOAD_RANGE(par, W, first) s16x8 W[G::FB]; _Pragma("unroll") for (int f_ = 0; f_ < G::FB; ++f_) W[f_] = BWFRAG(par, (first) + f_)

template <typename DT, int D, int DH, int ACT>
__global__ __launch_bounds__(512) void blocks_kernel(BlkArgs a) {
    typedef Geo<D> G;
    constexpr int NT = G::NT, KC = G::KC, H = D / DH, TPH = DH / 16;     // TPH: 16-feature tiles per head (2 or 3)
    constexpr int NB = G::NB, KB = G::KB, FB = G::FB;
    __shared__ __align__(16) uint2 ring[2][G::STAGE_U2];
    __shared__ uint2 kx[4][2][TPH][64];       // [env][row tile][feature tile of the head][lane]: K fragments
    __shared__ uint2 vx[4][2][TPH][64];       // V^T half fragments (this row tile's 4 keys per lane)
    extern __shared__ float4 bvl4[];          // fp32 vectors of every block
    const float* vlds = reinterpret_cast<const float*>(bvl4);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // in an SGPR: branches on it are scalar
    const int r16 = lane & 15, g = lane >> 4;
    const int el = wave >> 1, rt = wave & 1;
    const float scale_l2e = (DH == 32 ? 0.17677669529663688110f : 0.14433756729740644113f) * 1.44269504088896340736f;
    const int64_t ntiles = (a.B + 3) / 4;

    const uint2* img = a.frags;
    const uint2 z2 = make_uint2(0, 0);
    uint2 pr0a, pr0b, pr0c = z2, pr0d = z2, pr1a, pr1b, pr1c = z2, pr1d = z2;
    int pnext;
    {   // prologue: stage 0 -> ring slot 0; stages 1 and 2 in flight (every block has an even stage count >= 4)
#pragma unroll
        for (int u = 0; u < G::U2PT; ++u) ring[0][tid + 512 * u] = img[tid + 512 * u];
        pr1a = img[G::STAGE_U2 + tid]; pr1b = img[G::STAGE_U2 + tid + 512];
        if (G::U2PT >= 3) pr1c = img[G::STAGE_U2 + tid + 1024];
        if (G::U2PT == 4) pr1d = img[G::STAGE_U2 + tid + 1536];
        pr0a = img[2 * G::STAGE_U2 + tid]; pr0b = img[2 * G::STAGE_U2 + tid + 512];
        if (G::U2PT >= 3) pr0c = img[2 * G::STAGE_U2 + tid + 1024];
        if (G::U2PT == 4) pr0d = img[2 * G::STAGE_U2 + tid + 1536];
        pnext = 3 % a.total_stages;
        const int nv4 = a.n_layers * G::lv_size(a.F) / 4;
        for (int i = tid; i < nv4; i += 512) bvl4[i] = reinterpret_cast<const float4*>(a.vec)[i];
        blk_barrier();
    }

    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t env = tile * 4 + el;
        const int64_t envc = env < a.B ? env : a.B - 1;
        const int row = 16 * rt + r16;
        const bool row_ok = row < a.T;
        f32x4 x[NT];
        BFrag8 hf[KC];       // LayerNorm output as operand fragments
        BFrag8 of[KC];       // attention output fragments
        float kmask[2][4];   // additive key bias * log2(e) for keys 16*kt + 4g + i; -inf past T
        {
            const u16* xr = a.x_in + (envc * a.T + (row_ok ? row : 0)) * D;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint2 v = *reinterpret_cast<const uint2*>(xr + 16 * nt + 4 * g);
                x[nt][0] = row_ok ? DT::to_f((u16)(v.x & 0xffff)) : 0.f;
                x[nt][1] = row_ok ? DT::to_f((u16)(v.x >> 16)) : 0.f;
                x[nt][2] = row_ok ? DT::to_f((u16)(v.y & 0xffff)) : 0.f;
                x[nt][3] = row_ok ? DT::to_f((u16)(v.y >> 16)) : 0.f;
            }
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = 16 * kt + 4 * g + i;
                    kmask[kt][i] = key < a.T ? DT::to_f(a.key_bias[envc * a.T + key]) * 1.44269504088896340736f : -INFINITY;
                }
        }

        auto norm_to_frags = [&](const float* gptr, const float* bptr) __attribute__((always_inline)) {
            // one pass: var = E[x^2] - mean^2 clamped at 0 (python/beat_arena_env/csrc/layer_norm.cu:14-21)
            float s = 0.f, q = 0.f;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) { s += x[nt][i]; q = fmaf(x[nt][i], x[nt][i], q); }
            s += __shfl_xor(s, 16, WAVE); q += __shfl_xor(q, 16, WAVE);
            s += __shfl_xor(s, 32, WAVE); q += __shfl_xor(q, 32, WAVE);
            const float mean = s * (1.0f / D);
            const float rstd = rsqrtf(fmaxf(fmaf(-mean, mean, q * (1.0f / D)), 0.f) + 1e-5f);
            const float shift = -mean * rstd;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 gm = *reinterpret_cast<const float4*>(gptr + 16 * nt + 4 * g);
                const float4 bt = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
                const float y0 = fmaf(fmaf(x[nt][0], rstd, shift), gm.x, bt.x);
                const float y1 = fmaf(fmaf(x[nt][1], rstd, shift), gm.y, bt.y);
                const float y2 = fmaf(fmaf(x[nt][2], rstd, shift), gm.z, bt.z);
                const float y3 = fmaf(fmaf(x[nt][3], rstd, shift), gm.w, bt.w);
                hf[nt >> 1].w[(nt & 1) * 2] = bpack2<DT>(y0, y1);
                hf[nt >> 1].w[(nt & 1) * 2 + 1] = bpack2<DT>(y2, y3);
            }
        };
        auto add_bias = [&](const float* bptr) __attribute__((always_inline)) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 b = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
                x[nt][0] += b.x; x[nt][1] += b.y; x[nt][2] += b.z; x[nt][3] += b.w;
            }
        };
        auto store_rows = [&](u16* dst, int rows_per_env, int nrows_valid) __attribute__((always_inline)) {
            // this wave's rows < nrows_valid of its env, 4 consecutive features (8 bytes) per lane and tile
            if (env < a.B && row < nrows_valid) {
                u16* o = dst + (env * rows_per_env + row) * D;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    uint2 v;
                    v.x = bpack2<DT>(x[nt][0], x[nt][1]); v.y = bpack2<DT>(x[nt][2], x[nt][3]);
                    *reinterpret_cast<uint2*>(o + 16 * nt + 4 * g) = v;
                }
            }
        };

        // one block; in the pruned final block only row tile 0 carries queries.  `pruned` is a compile-time
        // constant so that the full blocks carry no branches around their MFMAs.
        auto layer = [&](int l, auto pruned_) __attribute__((always_inline)) {
            constexpr bool pruned = decltype(pruned_)::value;
            const float* lv = vlds + l * G::lv_size(a.F);
            const bool active = !pruned || rt == 0;          // wave-uniform
            if (pruned && a.x_res) store_rows(a.x_res, a.T, a.T);

            norm_to_frags(lv + G::LN1G, lv + G::LN1B);

            uint2 q[2][TPH];                                  // Q fragments, double-buffered by head parity

            // attention of head hd for this wave's 16 queries over the env's 32 key slots
            auto attention = [&](auto hd_) __attribute__((always_inline)) {
                constexpr int hd = decltype(hd_)::value;
                if (!active) return;
                f32x4 sc[2];
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    BFrag8 kf, qf;
                    kf.h[0] = kx[el][kt][0][lane]; kf.h[1] = kx[el][kt][1][lane];
                    qf.h[0] = q[hd & 1][0]; qf.h[1] = q[hd & 1][1];
                    sc[kt] = DT::mfma32(kf.v, qf.v, (f32x4){0.f, 0.f, 0.f, 0.f});
                    if (TPH == 3) {
                        // features 32..47: a K = 16 MFMA into its OWN accumulator (chaining it onto the
                        // 16x16x32 accumulator loses the first product on this hardware), summed on the VALU
                        BFrag4 k2, q2;
                        k2.h = kx[el][kt][TPH - 1][lane]; q2.h = q[hd & 1][TPH - 1];
                        const f32x4 s2 = DT::mfma16(k2.v, q2.v, (f32x4){0.f, 0.f, 0.f, 0.f});
#pragma unroll
                        for (int i = 0; i < 4; ++i) sc[kt][i] += s2[i];
                    }
                }
                float sv[2][4];
                float m = -INFINITY;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) { sv[kt][i] = fmaf(sc[kt][i], scale_l2e, kmask[kt][i]); m = fmaxf(m, sv[kt][i]); }
                m = fmaxf(m, __shfl_xor(m, 16, WAVE)); m = fmaxf(m, __shfl_xor(m, 32, WAVE));
                float sum = 0.f;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) { sv[kt][i] = __builtin_amdgcn_exp2f(sv[kt][i] - m); sum += sv[kt][i]; }
                sum += __shfl_xor(sum, 16, WAVE); sum += __shfl_xor(sum, 32, WAVE);
                const float inv = __builtin_amdgcn_rcpf(sum);
                BFrag8 pf;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    pf.w[2 * kt] = bpack2<DT>(sv[kt][0] * inv, sv[kt][1] * inv);
                    pf.w[2 * kt + 1] = bpack2<DT>(sv[kt][2] * inv, sv[kt][3] * inv);
                }
#pragma unroll
                for (int t = 0; t < TPH; ++t) {
                    BFrag8 vf;
                    vf.h[0] = vx[el][0][t][lane]; vf.h[1] = vx[el][1][t][lane];
                    const float4 bv = *reinterpret_cast<const float4*>(lv + G::BV + DH * hd + 16 * t + 4 * g);
                    const f32x4 o = DT::mfma32(vf.v, pf.v, (f32x4){bv.x, bv.y, bv.z, bv.w});
                    const int nt = hd * TPH + t;
                    of[nt >> 1].w[(nt & 1) * 2] = bpack2<DT>(o[0], o[1]);
                    of[nt >> 1].w[(nt & 1) * 2 + 1] = bpack2<DT>(o[2], o[3]);
                }
            };

            // ---- packed q|k|v projection: 3 * NT feature tiles in head-major order
            //      [q tiles | k tiles | v tiles] per head, two tiles per stage ----
            static_for<0, 3 * NT / 2>([&](auto st_) __attribute__((always_inline)) {
                constexpr int st = decltype(st_)::value;
                BADVANCE(st & 1);
                // a head whose last tile was computed in an earlier stage is complete in LDS after this barrier
                if constexpr (st > 0) {
                    constexpr int done = (2 * st) / (3 * TPH);        // heads complete before this stage's first tile
                    constexpr int done_prev = (2 * st - 2) / (3 * TPH);
                    if constexpr (done > done_prev) attention(std::integral_constant<int, done - 1>{});
                }
                f32x4 acc[2];
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const int j = 2 * st + ntl, hd = j / (3 * TPH), r = j % (3 * TPH), part = r / TPH, t = r % TPH;
                    float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (part < 2) b = *reinterpret_cast<const float4*>(lv + (part == 0 ? G::BQ : G::BK) + DH * hd + 16 * t + 4 * g);
                    acc[ntl] = (f32x4){b.x, b.y, b.z, b.w};
                }
#pragma unroll
                for (int half = 0; half < NB; ++half) {
                    BLOAD_BURST(st & 1, wf, half);                     // k chunks [half * KB, +KB) of both tiles
#pragma unroll
                    for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                        for (int ntl = 0; ntl < 2; ++ntl) {
                            const int c = half * KB + ci;
                            const int j = 2 * st + ntl, part = (j % (3 * TPH)) / TPH;
                            if (part == 0 && !active) continue;        // the pruned block needs no queries from row tile 1
                            const s16x8 w = wf[ntl * KB + ci];
                            if (part < 2) acc[ntl] = DT::mfma32(w, hf[c].v, acc[ntl]);
                            else acc[ntl] = DT::mfma32(hf[c].v, w, acc[ntl]);   // V^T: operand roles swapped
                        }
                }
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const int j = 2 * st + ntl, hd = j / (3 * TPH), r = j % (3 * TPH), part = r / TPH, t = r % TPH;
                    uint2 pk;
                    pk.x = bpack2<DT>(acc[ntl][0], acc[ntl][1]); pk.y = bpack2<DT>(acc[ntl][2], acc[ntl][3]);
                    if (part == 0) q[hd & 1][t] = pk;
                    else if (part == 1) kx[el][rt][t][lane] = pk;
                    else vx[el][rt][t][lane] = pk;
                }
            });

            // ---- output projection onto the residual (NT / 2 stages) ----
            if (active) add_bias(lv + G::BOUT);
            static_for<0, NT / 2>([&](auto st_) __attribute__((always_inline)) {
                constexpr int st = decltype(st_)::value;
                BADVANCE((3 * NT / 2 + st) & 1);
                if constexpr (st == 0) attention(std::integral_constant<int, H - 1>{});               // the last head completed in the previous stage
#pragma unroll
                for (int half = 0; half < NB; ++half) {
                    if (active) {            // idle waves of the pruned block leave the LDS bandwidth to the others
                        BLOAD_BURST((3 * NT / 2 + st) & 1, wf, half);
#pragma unroll
                        for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                            for (int ntl = 0; ntl < 2; ++ntl)
                                x[2 * st + ntl] = DT::mfma32(wf[ntl * KB + ci], of[half * KB + ci].v, x[2 * st + ntl]);
                    }
                }
            });

            // ---- LayerNorm + FFN: stage order W1(0), {W1(ch+1), W2(ch)}..., W2(last); the hidden of a
            //      32-unit chunk lives in two accumulators, activated and packed into one operand fragment ----
            constexpr int P0 = (3 * NT / 2 + NT / 2) & 1;              // stage parity at FFN entry (0: 2 * NT is even)
            static_assert(P0 == 0, "FFN stages start on an even stage");
            if (active) { norm_to_frags(lv + G::LN2G, lv + G::LN2B); add_bias(lv + G::b2(a.F)); }
            const int nch = a.F / 32;
            f32x4 accA[2];
            auto up = [&](int par, int ch, f32x4 (&acc)[2]) __attribute__((always_inline)) {
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const float4 b = *reinterpret_cast<const float4*>(lv + G::B1 + 32 * ch + 16 * ntl + 4 * g);
                    acc[ntl] = (f32x4){b.x, b.y, b.z, b.w};
                }
#pragma unroll
                for (int half = 0; half < NB; ++half) {
                    if (active) {
                        BLOAD_BURST(par, wf, half);
#pragma unroll
                        for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                            for (int ntl = 0; ntl < 2; ++ntl)
                                acc[ntl] = DT::mfma32(wf[ntl * KB + ci], hf[half * KB + ci].v, acc[ntl]);
                    }
                }
            };
            BADVANCE(0);
            up(0, 0, accA);
            for (int ch = 0; ch < nch; ++ch) {
                BFrag8 hid;
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    hid.w[ntl * 2] = bpack2<DT>(apply_act16<ACT>(accA[ntl][0]), apply_act16<ACT>(accA[ntl][1]));
                    hid.w[ntl * 2 + 1] = bpack2<DT>(apply_act16<ACT>(accA[ntl][2]), apply_act16<ACT>(accA[ntl][3]));
                }
                if (ch + 1 < nch) {
                    BADVANCE(1);
                    up(1, ch + 1, accA);
                    BADVANCE(0);
#pragma unroll
                    for (int half = 0; half < NB; ++half) {
                        if (active) {
                            BLOAD_RANGE(0, w2, half * FB);
#pragma unroll
                            for (int i = 0; i < FB; ++i) x[half * FB + i] = DT::mfma32(w2[i], hid.v, x[half * FB + i]);
                        }
                    }
                } else {
                    BADVANCE(1);
#pragma unroll
                    for (int half = 0; half < NB; ++half) {
                        if (active) {
                            BLOAD_RANGE(1, w2, half * FB);
#pragma unroll
                            for (int i = 0; i < FB; ++i) x[half * FB + i] = DT::mfma32(w2[i], hid.v, x[half * FB + i]);
                        }
                    }
                }
            }
        };
        const int n_full = a.n_queries > 0 ? a.n_layers - 1 : a.n_layers;
        for (int l = 0; l < n_full; ++l) layer(l, std::false_type{});
        if (a.n_queries > 0) layer(a.n_layers - 1, std::true_type{});
        if (a.n_queries > 0) { if (rt == 0) store_rows(a.x_out, a.n_queries, a.n_queries); }
        else store_rows(a.x_out, a.T, a.T);
    }
}



// ---- the same stack with ONE WAVE PER ENV ---------------------------------------------------------------------
// Mapping.  A wave owns both 16-row tiles of an env (all its <= 32 tokens) and carries their fp32 residual stream in
// registers; a workgroup is 8 waves = 8 envs, one workgroup per CU, two waves per SIMD in 256 registers each.
// Against blocks_kernel (a wave per row tile, an env a wave pair, 4 envs per workgroup):
//   * every weight fragment read from LDS feeds TWO MFMAs (one per row tile) instead of one, and a stage streamed from
//     L2 serves 8 envs instead of 4: half the LDS read instructions, barriers and stage loads per env;
//   * attention needs no LDS: a wave holds the K and V^T fragments of both key tiles of the head it just projected;
//   * stages go global -> LDS directly (global_load_lds_dwordx4, one 1 KB fragment per wave instruction) several
//     stages ahead into a ring of SLOTS stage slots: no register staging, depth bounded by LDS only;
//   * the row reductions of LayerNorm and softmax are lane-row swaps on the VALU, not shuffles through LDS.
// Per-row arithmetic, its order and the weight image are those of blocks_kernel: an env's output bits are the same.
// m0 (the LDS base of the transfer) is written without telling the compiler, which rejects reserved registers in a
// clobber list: nothing else in the kernel uses it.  No "memory" clobber: what orders these asynchronous LDS writes
// against the fragment reads is the vmcnt wait + barrier of the stage admission.  The instruction's immediate offset
// moves BOTH addresses of a transfer, the global one and the LDS one: a wave's second fragment of a stage is the one
// right after its first and costs no further scalar work.
__device__ __forceinline__ void env_ring_load(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr));
}
__device__ __forceinline__ void env_ring_load2(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024"
                 ::"v"(voff), "s"(sbase), "s"(lds_addr));
}
__device__ __forceinline__ void env_ring_load3(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024\n\t"
                 "global_load_lds_dwordx4 %0, %1 offset:2048" ::"v"(voff), "s"(sbase), "s"(lds_addr));
}

// The weight-stage ring of the one-wave-per-env kernels: stages of SF 1 KB fragments go global -> LDS directly, SLOTS
// stage slots deep.  Stages are entered in PAIRS (every block has an even number of them): one wait + barrier admits
// two stages and refills the two slots behind them, so all but those four slots may be in flight (AHEAD).  A loading
// wave moves FPW ADJACENT fragments of every stage (eight waves: SF = 8 one each; 12: six waves two each; 16: two each;
// four waves: 8: two each; 12: three each; 24: six each); image and ring are addressed by running byte offsets, no
// multiplies in the loop.
template <int SF_, int SLOTS_, int NW_ = 8> struct StageRing {
    static constexpr int NW = NW_, SF = SF_, SLOTS = SLOTS_, AHEAD = SLOTS - 4;
    static constexpr int FPW = (SF + NW - 1) / NW <= 1 ? 1 : SF % 2 == 0 && SF / 2 <= NW ? 2 : SF % 3 == 0 && SF / 3 <= NW ? 3 : 6;
    static constexpr int NLW = SF / FPW;               // FPW = 6: two transfers of three (the immediate offset ends at 4095)
    static constexpr uint32_t STAGE_BYTES = SF * 1024;
    static_assert(SLOTS >= 5 && FPW * NLW == SF && NLW <= NW && FPW * (AHEAD + 2) < 64, "fragment split; vmcnt is 6 bits");
    const uint4* ring;             // slot 0
    const char* wsrc;              // this wave's fragments of stage 0
    uint32_t wdst;                 // ... and their place in slot 0 (LDS byte address)
    uint32_t voff;                 // lane * 16
    uint32_t src_off, src_end;     // next stage to load, image length (bytes)
    uint32_t cur, prev;            // slot of the current stage and of the one before it (bytes from slot 0)
    bool loader;

    __device__ __forceinline__ void issue(uint32_t slot_off) {
        if (NLW == NW || loader) {
            if constexpr (FPW == 6) {
                env_ring_load3(voff, wsrc + src_off, wdst + slot_off);
                env_ring_load3(voff, wsrc + src_off + 3072, wdst + slot_off + 3072);
            } else if constexpr (FPW == 3) env_ring_load3(voff, wsrc + src_off, wdst + slot_off);
            else if constexpr (FPW == 2) env_ring_load2(voff, wsrc + src_off, wdst + slot_off);
            else env_ring_load(voff, wsrc + src_off, wdst + slot_off);
        }
        src_off = src_off + STAGE_BYTES == src_end ? 0 : src_off + STAGE_BYTES;
    }
    // SLOTS - 2 stages in flight (the host checks that the image is longer)
    __device__ __forceinline__ void start(const uint4* ring_, const void* img, int total_stages, int wave, int lane) {
        ring = ring_;
        wsrc = reinterpret_cast<const char*>(img) + wave * (FPW * 1024);
        wdst = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)const_cast<uint4*>(ring_) + wave * (FPW * 1024);
        voff = lane * 16;
        loader = wave < NLW;
        src_off = 0;
        src_end = (uint32_t)total_stages * STAGE_BYTES;
        cur = (SLOTS - 1) * STAGE_BYTES;
        prev = (SLOTS - 2) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < SLOTS - 2; ++i) issue(i * STAGE_BYTES);
    }
    // entry of the next stage (PARITY = its index in its block, mod 2): on return it is readable in slot `cur`
    template <int PARITY> __device__ __forceinline__ void admit() {
        const uint32_t older = prev;
        prev = cur;
        cur = cur + STAGE_BYTES == SLOTS * STAGE_BYTES ? 0 : cur + STAGE_BYTES;
        if constexpr (PARITY == 0) {
            // this wave's loads of this stage and the next have landed once at most the AHEAD younger stages' are
            // outstanding (loads retire in order; any other load or store in flight, or a wave that loads nothing,
            // only makes the wait stricter) ...
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(FPW * AHEAD) : "memory");
            blk_barrier();             // ... and every wave's have; every wave is done reading the two stages before this one
            issue(older);
            issue(prev);
        }
    }
    // fragment i of the current stage, this lane's 16 bytes
    __device__ __forceinline__ s16x8 frag(int i, int lane) const {
        return __builtin_bit_cast(s16x8, ring[(cur >> 4) + i * 64 + lane]);
    }
};
template <int D> struct EnvRing : StageRing<Geo<D>::SF, D == 128 ? 10 : 7> {};

template <typename DT, int D, int DH, int ACT>
__global__ __launch_bounds__(512, 1) void blocks_env_kernel(BlkArgs a) {
    typedef Geo<D> G;
    typedef EnvRing<D> R;
    constexpr int NW = R::NW;
    constexpr int NT = G::NT, KC = G::KC, H = D / DH, TPH = DH / 16;
    constexpr int NB = G::NB, KB = G::KB, SF = G::SF;
    // a stage is consumed in 2 * NB sub-bursts of KB fragments (a burst of blocks_kernel is two of them: the k chunks
    // [b * KB, +KB) of the stage's first tile, then of its second; in a W2 stage KB consecutive feature tiles)
    constexpr int NSUB = 2 * NB;
    static_assert(G::FB == 2 * KB, "a burst is two sub-bursts");
    extern __shared__ float4 bvl4[];          // fp32 vectors of every block, then the stage ring (1 KB aligned)
    const float* vlds = reinterpret_cast<const float*>(bvl4);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const float scale_l2e = (DH == 32 ? 0.17677669529663688110f : 0.14433756729740644113f) * 1.44269504088896340736f;
    const int64_t ntiles = (a.B + NW - 1) / NW;
    const int ring_off_u4 = (a.n_layers * G::lv_size(a.F) / 4 + 63) & ~63;
    const uint4* ring = reinterpret_cast<const uint4*>(bvl4) + ring_off_u4;
    R pipe;
    auto advance = [&](auto parity_) __attribute__((always_inline)) { pipe.template admit<decltype(parity_)::value>(); };
    typedef std::integral_constant<int, 0> Even;
    typedef std::integral_constant<int, 1> Odd;
    // sub-burst j of the current stage -> registers, then `body` on them
    auto sub = [&](auto j_, auto&& body) __attribute__((always_inline)) {
        constexpr int j = decltype(j_)::value;
        s16x8 w[KB];
#pragma unroll
        for (int f = 0; f < KB; ++f) w[f] = pipe.frag(j * KB + f, lane);
        body(w);
    };
    {   // prologue: SLOTS - 2 stages in flight (every stack has more), then the vectors
        pipe.start(ring, a.frags, a.total_stages, wave, lane);
        const int nv4 = a.n_layers * G::lv_size(a.F) / 4;
        for (int i = tid; i < nv4; i += NW * 64) bvl4[i] = reinterpret_cast<const float4*>(a.vec)[i];
        blk_barrier();
    }

    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t env = tile * NW + wave;
        const int64_t envc = env < a.B ? env : a.B - 1;
        f32x4 x[2][NT];
        BFrag8 hf[2][KC];    // LayerNorm output as operand fragments
        BFrag8 of[2][KC];    // attention output fragments
        float kmask[2][4];   // additive key bias * log2(e) for keys 16*kt + 4g + i; -inf past T
        // the tile's own loads are all issued, then waited for ONCE, with the wait the compiler can see (vmcnt(0); expcnt /
        // lgkmcnt at their maxima).  It does not know of the ring's loads: wherever it later met a value of its own still
        // in flight - or reused such a register - it would wait for every outstanding load, i.e. drain the ring in mid-tile.
        uint2 raw[2][NT];
        u16 kraw[2][4];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int row = 16 * rt + r16;
            const u16* xr = a.x_in + (envc * a.T + (row < a.T ? row : 0)) * D;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) raw[rt][nt] = *reinterpret_cast<const uint2*>(xr + 16 * nt + 4 * g);
        }
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = 16 * kt + 4 * g + i;
                kraw[kt][i] = a.key_bias[envc * a.T + (key < a.T ? key : 0)];
            }
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const bool row_ok = 16 * rt + r16 < a.T;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint32_t lo = row_ok ? raw[rt][nt].x : 0u, hi = row_ok ? raw[rt][nt].y : 0u;      // 0 bits = +0.0
                x[rt][nt][0] = DT::to_f((u16)(lo & 0xffff)); x[rt][nt][1] = DT::to_f((u16)(lo >> 16));
                x[rt][nt][2] = DT::to_f((u16)(hi & 0xffff)); x[rt][nt][3] = DT::to_f((u16)(hi >> 16));
            }
        }
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                kmask[kt][i] = 16 * kt + 4 * g + i < a.T ? DT::to_f(kraw[kt][i]) * 1.44269504088896340736f : -INFINITY;

        // LayerNorm of both row tiles (of row tile 0 only: `both` false) -> operand fragments; the statistics of the two
        // tiles go through the lane-row butterfly together
        auto norm_to_frags = [&](bool both, const float* gptr, const float* bptr) __attribute__((always_inline)) {
            // one pass: var = E[x^2] - mean^2 clamped at 0 (python/beat_arena_env/csrc/layer_norm.cu:14-21)
            float s[2] = {0.f, 0.f}, q[2] = {0.f, 0.f};
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt == 1 && !both) break;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) { s[rt] += x[rt][nt][i]; q[rt] = fmaf(x[rt][nt][i], x[rt][nt][i], q[rt]); }
            }
            rows_reduce2(s[0], q[0], OpAdd());
            if (both) rows_reduce2(s[1], q[1], OpAdd());
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt == 1 && !both) break;
                const float mean = s[rt] * (1.0f / D);
                const float rstd = rsqrtf(fmaxf(fmaf(-mean, mean, q[rt] * (1.0f / D)), 0.f) + 1e-5f);
                const float shift = -mean * rstd;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float4 gm = *reinterpret_cast<const float4*>(gptr + 16 * nt + 4 * g);
                    const float4 bt = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
                    const float y0 = fmaf(fmaf(x[rt][nt][0], rstd, shift), gm.x, bt.x);
                    const float y1 = fmaf(fmaf(x[rt][nt][1], rstd, shift), gm.y, bt.y);
                    const float y2 = fmaf(fmaf(x[rt][nt][2], rstd, shift), gm.z, bt.z);
                    const float y3 = fmaf(fmaf(x[rt][nt][3], rstd, shift), gm.w, bt.w);
                    hf[rt][nt >> 1].w[(nt & 1) * 2] = bpack2<DT>(y0, y1);
                    hf[rt][nt >> 1].w[(nt & 1) * 2 + 1] = bpack2<DT>(y2, y3);
                }
            }
        };
        auto add_bias = [&](auto rt_, const float* bptr) __attribute__((always_inline)) {
            constexpr int rt = decltype(rt_)::value;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 b = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
                x[rt][nt][0] += b.x; x[rt][nt][1] += b.y; x[rt][nt][2] += b.z; x[rt][nt][3] += b.w;
            }
        };
        auto store_rows = [&](auto rt_, u16* dst, int rows_per_env, int nrows_valid) __attribute__((always_inline)) {
            constexpr int rt = decltype(rt_)::value;
            const int row = 16 * rt + r16;
            if (env < a.B && row < nrows_valid) {
                u16* o = dst + (env * rows_per_env + row) * D;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    uint2 v;
                    v.x = bpack2<DT>(x[rt][nt][0], x[rt][nt][1]); v.y = bpack2<DT>(x[rt][nt][2], x[rt][nt][3]);
                    *reinterpret_cast<uint2*>(o + 16 * nt + 4 * g) = v;
                }
            }
        };
        typedef std::integral_constant<int, 0> T0;
        typedef std::integral_constant<int, 1> T1;

        // one block; the pruned final block computes queries, output projection and FFN for row tile 0 only (keys and
        // values of both).  `pruned` is a compile-time constant: the full blocks carry no branches around their MFMAs.
        auto layer = [&](int l, auto pruned_) __attribute__((always_inline)) {
            constexpr bool pruned = decltype(pruned_)::value;
            constexpr int QT = pruned ? 1 : 2;                 // query row tiles
            const float* lv = vlds + l * G::lv_size(a.F);
            if (pruned && a.x_res) { store_rows(T0(), a.x_res, a.T, a.T); store_rows(T1(), a.x_res, a.T, a.T); }

            norm_to_frags(true, lv + G::LN1G, lv + G::LN1B);

            uint2 q[2][2][TPH];                                // Q fragments [head parity][row tile][feature tile]
            uint2 kk[2][TPH], vv[2][TPH];                      // K, V^T fragments of the head in flight [key tile][feature tile]

            // attention of head hd: the env's (up to) 32 queries over its 32 key slots, both query tiles together
            auto attention = [&](auto hd_) __attribute__((always_inline)) {
                constexpr int hd = decltype(hd_)::value;
                float sv[2][2][4], m[2], sum[2];
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) {
                    f32x4 sc[2];
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt) {
                        BFrag8 kf, qf;
                        kf.h[0] = kk[kt][0]; kf.h[1] = kk[kt][1];
                        qf.h[0] = q[hd & 1][qt][0]; qf.h[1] = q[hd & 1][qt][1];
                        sc[kt] = DT::mfma32(kf.v, qf.v, (f32x4){0.f, 0.f, 0.f, 0.f});
                        if (TPH == 3) {
                            // features 32..47: a K = 16 MFMA into its OWN accumulator (chaining it onto the
                            // 16x16x32 accumulator loses the first product on this hardware), summed on the VALU
                            BFrag4 k2, q2;
                            k2.h = kk[kt][TPH - 1]; q2.h = q[hd & 1][qt][TPH - 1];
                            const f32x4 s2 = DT::mfma16(k2.v, q2.v, (f32x4){0.f, 0.f, 0.f, 0.f});
#pragma unroll
                            for (int i = 0; i < 4; ++i) sc[kt][i] += s2[i];
                        }
                    }
                    m[qt] = -INFINITY;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) { sv[qt][kt][i] = fmaf(sc[kt][i], scale_l2e, kmask[kt][i]); m[qt] = fmaxf(m[qt], sv[qt][kt][i]); }
                }
                if (QT == 1) m[1] = m[0];
                rows_reduce2(m[0], m[1], OpMax());
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) {
                    sum[qt] = 0.f;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) { sv[qt][kt][i] = __builtin_amdgcn_exp2f(sv[qt][kt][i] - m[qt]); sum[qt] += sv[qt][kt][i]; }
                }
                if (QT == 1) sum[1] = sum[0];
                rows_reduce2(sum[0], sum[1], OpAdd());
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) {
                    const float inv = __builtin_amdgcn_rcpf(sum[qt]);
                    BFrag8 pf;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt) {
                        pf.w[2 * kt] = bpack2<DT>(sv[qt][kt][0] * inv, sv[qt][kt][1] * inv);
                        pf.w[2 * kt + 1] = bpack2<DT>(sv[qt][kt][2] * inv, sv[qt][kt][3] * inv);
                    }
#pragma unroll
                    for (int t = 0; t < TPH; ++t) {
                        BFrag8 vf;
                        vf.h[0] = vv[0][t]; vf.h[1] = vv[1][t];
                        const float4 bv = *reinterpret_cast<const float4*>(lv + G::BV + DH * hd + 16 * t + 4 * g);
                        const f32x4 o = DT::mfma32(vf.v, pf.v, (f32x4){bv.x, bv.y, bv.z, bv.w});
                        const int nt = hd * TPH + t;
                        of[qt][nt >> 1].w[(nt & 1) * 2] = bpack2<DT>(o[0], o[1]);
                        of[qt][nt >> 1].w[(nt & 1) * 2 + 1] = bpack2<DT>(o[2], o[3]);
                    }
                }
            };

            // ---- packed q|k|v projection: 3 * NT feature tiles in head-major order [q | k | v] per head, two per stage ----
            static_for<0, 3 * NT / 2>([&](auto st_) __attribute__((always_inline)) {
                constexpr int st = decltype(st_)::value;
                advance(std::integral_constant<int, st & 1>{});
                // a head whose last tile was computed in an earlier stage is complete now: its attention runs before
                // this stage's results overwrite the K / V registers (a stage that straddles two heads holds the LAST
                // tile of one and the FIRST - a query tile, double-buffered by head parity - of the next)
                if constexpr (st > 0) {
                    constexpr int done = (2 * st) / (3 * TPH);
                    constexpr int done_prev = (2 * st - 2) / (3 * TPH);
                    if constexpr (done > done_prev) attention(std::integral_constant<int, done - 1>{});
                }
                f32x4 acc[2][2];                                 // [tile of the stage][row tile]
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const int j = 2 * st + ntl, hd = j / (3 * TPH), r = j % (3 * TPH), part = r / TPH, t = r % TPH;
                    float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (part < 2) b = *reinterpret_cast<const float4*>(lv + (part == 0 ? G::BQ : G::BK) + DH * hd + 16 * t + 4 * g);
                    acc[ntl][0] = (f32x4){b.x, b.y, b.z, b.w}; acc[ntl][1] = acc[ntl][0];
                }
                static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                    constexpr int half = decltype(j_)::value / 2, ntl = decltype(j_)::value % 2;    // k chunks [half * KB, +KB) of tile ntl
                    sub(j_, [&](const s16x8 (&wf)[KB]) __attribute__((always_inline)) {
#pragma unroll
                        for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                            for (int rt = 0; rt < 2; ++rt) {
                                const int c = half * KB + ci;
                                const int j = 2 * st + ntl, part = (j % (3 * TPH)) / TPH;
                                if (part == 0 && rt >= QT) continue;     // the pruned block needs no queries from row tile 1
                                if (part < 2) acc[ntl][rt] = DT::mfma32(wf[ci], hf[rt][c].v, acc[ntl][rt]);
                                else acc[ntl][rt] = DT::mfma32(hf[rt][c].v, wf[ci], acc[ntl][rt]);   // V^T: operand roles swapped
                            }
                    });
                });
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt) {
                        const int j = 2 * st + ntl, hd = j / (3 * TPH), r = j % (3 * TPH), part = r / TPH, t = r % TPH;
                        if (part == 0 && rt >= QT) continue;
                        uint2 pk;
                        pk.x = bpack2<DT>(acc[ntl][rt][0], acc[ntl][rt][1]); pk.y = bpack2<DT>(acc[ntl][rt][2], acc[ntl][rt][3]);
                        if (part == 0) q[hd & 1][rt][t] = pk;
                        else if (part == 1) kk[rt][t] = pk;
                        else vv[rt][t] = pk;
                    }
            });

            // ---- output projection onto the residual (NT / 2 stages) ----
            add_bias(T0(), lv + G::BOUT);
            if (!pruned) add_bias(T1(), lv + G::BOUT);
            static_for<0, NT / 2>([&](auto st_) __attribute__((always_inline)) {
                constexpr int st = decltype(st_)::value;
                advance(std::integral_constant<int, st & 1>{});
                if constexpr (st == 0) attention(std::integral_constant<int, H - 1>{});      // the last head completed in the previous stage
                static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                    constexpr int half = decltype(j_)::value / 2, ntl = decltype(j_)::value % 2;
                    sub(j_, [&](const s16x8 (&wf)[KB]) __attribute__((always_inline)) {
#pragma unroll
                        for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                            for (int qt = 0; qt < QT; ++qt)
                                x[qt][2 * st + ntl] = DT::mfma32(wf[ci], of[qt][half * KB + ci].v, x[qt][2 * st + ntl]);
                    });
                });
            });

            // ---- LayerNorm + FFN: stage order W1(0), {W1(ch+1), W2(ch)}..., W2(last); the hidden of a 32-unit chunk
            //      lives in two accumulators per row tile, activated and packed into one operand fragment ----
            norm_to_frags(!pruned, lv + G::LN2G, lv + G::LN2B);
            add_bias(T0(), lv + G::b2(a.F));
            if (!pruned) add_bias(T1(), lv + G::b2(a.F));
            const int nch = a.F / 32;
            f32x4 acc[2][2];                                     // [tile of the chunk][row tile]
            auto up = [&](int ch) __attribute__((always_inline)) {
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const float4 b = *reinterpret_cast<const float4*>(lv + G::B1 + 32 * ch + 16 * ntl + 4 * g);
                    acc[ntl][0] = (f32x4){b.x, b.y, b.z, b.w}; acc[ntl][1] = acc[ntl][0];
                }
                static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                    constexpr int half = decltype(j_)::value / 2, ntl = decltype(j_)::value % 2;
                    sub(j_, [&](const s16x8 (&wf)[KB]) __attribute__((always_inline)) {
#pragma unroll
                        for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                            for (int qt = 0; qt < QT; ++qt)
                                acc[ntl][qt] = DT::mfma32(wf[ci], hf[qt][half * KB + ci].v, acc[ntl][qt]);
                    });
                });
            };
            static_assert((3 * NT / 2) % 2 == 0 && (NT / 2) % 2 == 0, "the FFN starts on an even stage");
            advance(Even{});
            up(0);
            for (int ch = 0; ch < nch; ++ch) {
                BFrag8 hid[2];
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
#pragma unroll
                    for (int ntl = 0; ntl < 2; ++ntl) {
                        hid[qt].w[ntl * 2] = bpack2<DT>(apply_act16<ACT>(acc[ntl][qt][0]), apply_act16<ACT>(acc[ntl][qt][1]));
                        hid[qt].w[ntl * 2 + 1] = bpack2<DT>(apply_act16<ACT>(acc[ntl][qt][2]), apply_act16<ACT>(acc[ntl][qt][3]));
                    }
                // stage parities: W1(0) even, then {W1(ch + 1) odd, W2(ch) even} ..., W2(last) odd
                if (ch + 1 < nch) { advance(Odd{}); up(ch + 1); advance(Even{}); }
                else advance(Odd{});
                static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                    constexpr int j = decltype(j_)::value;           // feature tiles [j * KB, +KB)
                    sub(j_, [&](const s16x8 (&w2)[KB]) __attribute__((always_inline)) {
#pragma unroll
                        for (int i = 0; i < KB; ++i)
#pragma unroll
                            for (int qt = 0; qt < QT; ++qt) x[qt][j * KB + i] = DT::mfma32(w2[i], hid[qt].v, x[qt][j * KB + i]);
                    });
                });
            }
        };
        const int n_full = a.n_queries > 0 ? a.n_layers - 1 : a.n_layers;
        for (int l = 0; l < n_full; ++l) layer(l, std::false_type{});
        if (a.n_queries > 0) layer(a.n_layers - 1, std::true_type{});
        if (a.n_queries > 0) store_rows(T0(), a.x_out, a.n_queries, a.n_queries);
        else { store_rows(T0(), a.x_out, a.T, a.T); store_rows(T1(), a.x_out, a.T, a.T); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // no transfer into LDS may outlive the workgroup
    blk_barrier();
}

// ---- weight image ------------------------------------------------------------------
struct BlkPackArgs {
    bsrl_blocks_params p;
    void* frags; float* vec;
    int n_layers, F;
};
__device__ __forceinline__ int bperm_k(int c, int gg, int j) { return 32 * c + 4 * gg + (j & 3) + (j >> 2) * 16; }

// one wave per fragment, one lane per 16-byte slot
template <typename DT, int D, int DH>
__global__ __launch_bounds__(256) void blocks_pack_frags_kernel(BlkPackArgs a) {
    typedef Geo<D> G;
    constexpr int NT = G::NT, KC = G::KC, SF = G::SF, TPH = DH / 16;
    const int lane = threadIdx.x & 63;
    const int lfr = G::layer_stages(a.F) * SF;                 // fragments per block
    const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= a.n_layers * lfr) return;
    const int n16 = lane & 15, gg = lane >> 4;
    const int l = f / lfr, r = f % lfr;
    const auto& b = a.p.blk[l];
    const float* src; int ld, n, kbase = 0, c;
    // inside a stage of two feature tiles the fragments are ordered (burst, tile, k chunk of the burst):
    // consecutive runs of FB fragments are what a consumer reads together
    auto split = [&](int i, int& ntl, int& cc) {
        const int burst = i / G::FB, rem = i % G::FB;
        ntl = rem / G::KB; cc = burst * G::KB + rem % G::KB;
    };
    if (r < 3 * NT * KC) {
        int ntl; split(r % SF, ntl, c);
        const int j = 2 * (r / SF) + ntl, hd = j / (3 * TPH), rr = j % (3 * TPH), part = rr / TPH, t = rr % TPH;
        src = part == 0 ? b.q_w : part == 1 ? b.k_w : b.v_w;
        ld = D; n = DH * hd + 16 * t + n16;
    } else if (r < 4 * NT * KC) {
        const int r2 = r - 3 * NT * KC;
        int ntl; split(r2 % SF, ntl, c);
        src = b.out_w; ld = D; n = 16 * (2 * (r2 / SF) + ntl) + n16;
    } else {
        const int r3 = r - 4 * NT * KC, s3 = r3 / SF, i = r3 % SF, nch = a.F / 32;
        bool upw; int ch;
        if (s3 == 0) { upw = true; ch = 0; }
        else if (s3 == 2 * nch - 1) { upw = false; ch = nch - 1; }
        else { upw = ((s3 - 1) & 1) == 0; ch = (s3 - 1) / 2 + (upw ? 1 : 0); }
        if (upw) { int ntl; split(i, ntl, c); src = b.ffn0_w; ld = D; n = 32 * ch + 16 * ntl + n16; }
        else { src = b.ffn2_w; ld = a.F; n = 16 * i + n16; c = 0; kbase = 32 * ch; }
    }
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[(int64_t)n * ld + kbase + bperm_k(c, gg, j)];
    uint4 o;
    o.x = bpack2<DT>(v[0], v[1]); o.y = bpack2<DT>(v[2], v[3]); o.z = bpack2<DT>(v[4], v[5]); o.w = bpack2<DT>(v[6], v[7]);
    static_cast<uint4*>(a.frags)[(int64_t)f * 64 + lane] = o;
}

template <int D>
__global__ __launch_bounds__(256) void blocks_pack_vec_kernel(BlkPackArgs a) {
    typedef Geo<D> G;
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int lvs = G::lv_size(a.F);
    if (i >= a.n_layers * lvs) return;
    const int l = i / lvs, r = i % lvs;
    const auto& b = a.p.blk[l];
    float v;
    if (r < G::B1) {
        const float* srcs[8] = {b.ln_attn_w, b.ln_attn_b, b.q_b, b.k_b, b.v_b, b.out_b, b.ln_ffn_w, b.ln_ffn_b};
        v = srcs[r / D][r % D];
    } else if (r < G::b2(a.F)) v = b.ffn0_b[r - G::B1];
    else v = b.ffn2_b[r - G::b2(a.F)];
    a.vec[i] = v;
}

constexpr int LDS_STATIC_MAX = 2 * 16 * 1024 + 2 * 4 * 2 * 3 * 64 * 8;      // upper bound of ring + K/V exchange over the shapes
constexpr int LDS_BUDGET = 160 * 1024;

bool blocks_shape_ok(const bsrl_blocks_desc* d) {
    if (!d) return false;
    const bool geo = (d->d == 128 && d->n_heads == 4) || (d->d == 192 && d->n_heads == 4) || (d->d == 256 && d->n_heads == 8);
    if (!geo || d->T < 1 || d->T > 32 || d->ffn <= 0 || d->ffn % 32 != 0 || d->ffn < 64 || d->n_layers < 1 ||
        d->n_layers > BSRL_MAX_LAYERS || (d->dtype != BSRL_F16 && d->dtype != BSRL_BF16) ||
        (d->act != BSRL_ACT_RELU && d->act != BSRL_ACT_GELU) || d->n_queries < 0 || d->n_queries > 16 || d->n_queries > d->T)
        return false;
    const int64_t vec_bytes = (int64_t)d->n_layers * (9 * d->d + d->ffn) * 4;
    return vec_bytes + LDS_STATIC_MAX <= LDS_BUDGET;
}
int64_t blocks_stages(const bsrl_blocks_desc* d) {
    return (int64_t)d->n_layers * (d->d == 128 ? Geo<128>::layer_stages(d->ffn) : d->d == 192 ? Geo<192>::layer_stages(d->ffn) : Geo<256>::layer_stages(d->ffn));
}
int64_t blocks_frag_bytes(const bsrl_blocks_desc* d) { return blocks_stages(d) * (d->d / 16) * 1024; }

template <typename DT, int D, int DH>
void pack_launch(const BlkPackArgs& pa, int64_t nfrags, hipStream_t st) {
    hipLaunchKernelGGL((blocks_pack_frags_kernel<DT, D, DH>), dim3((unsigned)((nfrags + 3) / 4)), dim3(256), 0, st, pa);
    const int nvec = pa.n_layers * Geo<D>::lv_size(pa.F);
    hipLaunchKernelGGL(blocks_pack_vec_kernel<D>, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, st, pa);
}

// dynamic LDS of the env-per-wave kernel: vectors (rounded to 1 KB) + ring
template <int D> size_t env_dyn_bytes(int n_layers, int F) {
    return (size_t)((n_layers * Geo<D>::lv_size(F) / 4 + 63) & ~63) * 16 + (size_t)EnvRing<D>::SLOTS * EnvRing<D>::STAGE_BYTES;
}
// The env-per-wave kernel runs where a wave's state fits 256 registers (d = 128 and 192: at d = 256 it would spill
// several hundred values), the vectors and the stage ring fit a workgroup's LDS, and the stack is at least as long as
// the ring; the wave-pair kernel otherwise.
template <int D> bool env_kernel_ok(const BlkArgs& a) {
    if (D == 256) return false;
    return env_dyn_bytes<D>(a.n_layers, a.F) + 1024 <= (size_t)LDS_BUDGET && a.total_stages >= EnvRing<D>::SLOTS && a.total_stages % 2 == 0;
}

template <typename DT, int D, int DH, int ACT>
int fwd_launch(const BlkArgs& a, int cus, hipStream_t st) {
    if constexpr (D != 256) {
        // ... and the batch fills the CUs with 8-env tiles: up to 4 envs per CU the wave-pair kernel's 4-env tiles
        // spread over twice as many CUs (both kernels produce the same bits for an env)
        if (env_kernel_ok<D>(a) && a.B > 4 * (int64_t)cus) {
            const size_t dyn = env_dyn_bytes<D>(a.n_layers, a.F);
            const int64_t ntiles = (a.B + EnvRing<D>::NW - 1) / EnvRing<D>::NW;
            auto kern = blocks_env_kernel<DT, D, DH, ACT>;
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess)
                return BSRL_UNSUPPORTED;
            hipLaunchKernelGGL(kern, dim3((unsigned)(ntiles < cus ? ntiles : cus)), dim3(EnvRing<D>::NW * 64), dyn, st, a);
            return BSRL_OK;
        }
    }
    const size_t dyn = (size_t)a.n_layers * Geo<D>::lv_size(a.F) * sizeof(float);
    const int64_t ntiles = (a.B + 3) / 4;
    const dim3 grid((unsigned)(ntiles < cus ? ntiles : cus));
    auto kern = blocks_kernel<DT, D, DH, ACT>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess)
        return BSRL_UNSUPPORTED;
    hipLaunchKernelGGL(kern, grid, dim3(512), dyn, st, a);
    return BSRL_OK;
}

// ---- the FFN half of a block as a kernel of its own: xo = x + act(h2 W0^T + b0) W2^T + b2 (+ LayerNorm) ------------
// The FFN phase of blocks_env_kernel on plain rows: a wave owns 32 rows (two 16-row tiles; fp32 accumulator and the
// LayerNorm-ed input as operand fragments in registers), a workgroup is 4 waves = 128 rows, two per CU (d = 256: 8 waves, one); the
// weight chunks stream through the same direct-to-LDS ring from a pre-permuted image (stage order W1(0), {W1(ch+1),
// W2(ch)}..., W2(last), admitted in pairs), every fragment feeds both row tiles, the 32-unit hidden chunk lives in
// accumulators and goes into the down-projection as one operand fragment.  Rounding points are those of the
// reference's fused kernel (python/beat_arena_env/csrc/fused_ffn.cu:551-619): hidden rounded once, fp32 accumulate,
// xo rounded once, LayerNorm statistics on the ROUNDED xo, ho rounded once.
struct FfnArgs {
    const uint2* frags; const float* vec;        // image: 2 * F / 32 stages, then b0 (F) | b2 (d) fp32
    const u16* x; const u16* h2; u16* xo; u16* ho; u16* hid;      // hid: (rows, F) activated hidden for a backward, or NULL
    const float* ln_w; const float* ln_b; float eps;
    int64_t rows; int F, total_stages;
    // the attention-side tail in front of the FFN (PROJ instantiations): h2 is then the attention output, the image
    // opens with d / 32 output-projection stages, vec continues with the projection bias
    const float* ln2_w; const float* ln2_b; float eps2;
    // ... and a projection of the LayerNorm-ed output behind it (PROJ, with LN): qo (rows, 32 * nq) = ho Wn^T + bn, as nq
    // more stages of the up-projection's form after the FFN stages (vec continues with bn); ho itself is stored only
    // when the pointer is given
    u16* qo; int nq;
};

// Eight waves, one workgroup per CU - or four waves, TWO workgroups per CU (d = 128 / 192, where two rings fit): the
// waves of a workgroup walk the ring in lockstep, so all of them load and store their rows at the same time with
// nothing to run meanwhile; a second, independent workgroup drifts out of phase and computes through it.
// d = 384: a wave's state (fp32 accumulator 192 registers, input fragments 96) wants the whole register file of a SIMD:
// four waves, ONE workgroup per CU, 512 registers each; stages of 24 KB.
// (XS: one more slot where the vectors leave room for it - a stage more in flight behind the pair being consumed)
template <int D, int NW, int XS = 0> struct FfnRing : StageRing<Geo<D>::SF, (NW == 8 ? (D == 128 ? 10 : D == 192 ? 7 : 6) : (D == 128 ? 8 : D == 192 ? 6 : 5)) + XS, NW> {};
template <int D, int NW> constexpr int ffn_wgs_per_cu() { return D == 384 ? 1 : 8 / NW; }

// PROJ (d = 384): the rest of the block's attention side in front of the FFN, in the same registers -
//   x1 = x + att Wo^T + bo (rounded once),  h2 = LayerNorm(x1; ln2) (rounded once),  then the FFN of (x1, h2) as above -
// what the output-projection kernel and the LayerNorm kernel between them would do through memory (three round trips
// of the stream).  The projection runs as d / 32 more stages of the down-projection's form (the attention output's
// operand fragments in place of the hidden chunk); the rounded x1 and h2 never leave the registers: a lane's four
// features of an accumulator tile are half of an operand fragment of the up-projection.
// LEAD (a PROJ instantiation with LN): nothing but the last phase - qo = LayerNorm(x) Wn^T + bn; the image holds the nq
// projection stages only (F = 0), h2 is not read, xo is not written.
template <typename DT, int D, int ACT, bool LN, bool SAVE, int NW_, int XS, bool PROJ = false, bool LEAD = false>
__global__ __launch_bounds__(NW_ * 64, (ffn_wgs_per_cu<D, NW_>())) void ffn_rows_kernel(FfnArgs a) {
    typedef Geo<D> G;
    typedef FfnRing<D, NW_, XS> R;
    static_assert(!PROJ || (D == 384 && !SAVE), "the projection form exists for the register-pipelined d = 384 kernel");
    static_assert(!LEAD || (PROJ && LN), "the lead form is the projection form's last phase");
    constexpr int NW = R::NW, NT = G::NT, KC = G::KC, NB = G::NB, KB = G::KB, NSUB = 2 * NB;
    extern __shared__ float4 bvl4[];          // b0 (F) | b2 (d) | ln_w (d) | ln_b (d), then the stage ring (1 KB aligned)
    float* vlds = reinterpret_cast<float*>(bvl4);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int nvec = a.F + (PROJ ? 6 * D + 32 * a.nq : 3 * D);         // PROJ: ... | bo (d) | ln2_w (d) | ln2_b (d) | bn (32 nq)
    const int ring_off_u4 = (nvec / 4 + 63) & ~63;
    const uint4* ring = reinterpret_cast<const uint4*>(bvl4) + ring_off_u4;
    const float* B1 = vlds; const float* B2 = vlds + a.F; const float* LNG = B2 + D; const float* LNB = LNG + D;
    const float* BO = LNB + D; const float* LN2G = BO + D; const float* LN2B = LN2G + D; const float* BN = LN2B + D;
    // WIDE (d = 384): the weight rows of an accumulator-tile PAIR are ordered so that a lane's four features of tile
    // 2p and its four of tile 2p + 1 are EIGHT CONSECUTIVE features, 32 p + 8 g + 0..7 (A row m of tile i is feature
    // 32 (i / 2) + 8 (m / 4) + 4 (i % 2) + m % 4): rows come in and leave in 16-byte pieces, 64 contiguous bytes per
    // row and instruction instead of 32, and both an input row's and a LayerNorm output's operand fragment hold their k
    // values in natural order.  foff(nt): first feature of the lane's four in tile nt.
    constexpr bool WIDE = D == 384;
    auto foff = [&](int nt) __attribute__((always_inline)) { return WIDE ? 32 * (nt >> 1) + 8 * g + 4 * (nt & 1) : 16 * nt + 4 * g; };
    const int64_t ntiles = (a.rows + NW * 32 - 1) / (NW * 32);

    R pipe;
    auto advance = [&](auto parity_) __attribute__((always_inline)) { pipe.template admit<decltype(parity_)::value>(); };
    typedef std::integral_constant<int, 0> Even;
    typedef std::integral_constant<int, 1> Odd;
    auto sub = [&](auto j_, auto&& body) __attribute__((always_inline)) {
        constexpr int j = decltype(j_)::value;
        s16x8 w[KB];
#pragma unroll
        for (int f = 0; f < KB; ++f) w[f] = pipe.frag(j * KB + f, lane);
        body(w);
    };
    {   // prologue: SLOTS - 2 stages in flight (the host checks that the image is longer), then the vectors
        pipe.start(ring, a.frags, a.total_stages, wave, lane);
        for (int i = tid; i < a.F + D; i += NW * 64) vlds[i] = a.vec[i];
        if (LN) for (int i = tid; i < D; i += NW * 64) { vlds[a.F + D + i] = a.ln_w[i]; vlds[a.F + 2 * D + i] = a.ln_b[i]; }
        if (PROJ) for (int i = tid; i < D; i += NW * 64) {
            vlds[a.F + 3 * D + i] = a.vec[a.F + D + i]; vlds[a.F + 4 * D + i] = a.ln2_w[i]; vlds[a.F + 5 * D + i] = a.ln2_b[i];
        }
        if (PROJ) for (int i = tid; i < 32 * a.nq; i += NW * 64) vlds[a.F + 6 * D + i] = a.vec[a.F + 2 * D + i];
        blk_barrier();
    }

    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t row0 = (tile * NW + wave) * 32;
        f32x4 x[2][NT];
        BFrag8 hf[2][KC];
        if constexpr (D == 384) {
            // every load of the tile issued at once - x row tile 0, x row tile 1, then h2 -, and the compiler's own waits
            // (it counts its loads, not the ring's transfers, which only makes them stricter) let each conversion start
            // as its rows land: one memory latency per tile, not one per array
            uint4 rx[2][NT / 2];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                int64_t row = row0 + 16 * rt + r16; row = row < a.rows ? row : a.rows - 1;
                const u16* xr = a.x + row * D;
#pragma unroll
                for (int p = 0; p < NT / 2; ++p) rx[rt][p] = *reinterpret_cast<const uint4*>(xr + 32 * p + 8 * g);
            }
            if constexpr (!LEAD)
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                int64_t row = row0 + 16 * rt + r16; row = row < a.rows ? row : a.rows - 1;
                const u16* hr = a.h2 + row * D;
#pragma unroll
                for (int c = 0; c < KC; ++c) {
                    const uint4 r4 = *reinterpret_cast<const uint4*>(hr + 32 * c + 8 * g);
                    hf[rt][c].h[0] = make_uint2(r4.x, r4.y); hf[rt][c].h[1] = make_uint2(r4.z, r4.w);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float4 b = *reinterpret_cast<const float4*>((PROJ ? BO : B2) + foff(nt));
                    const uint32_t lo = (nt & 1) ? rx[rt][nt >> 1].z : rx[rt][nt >> 1].x, hi = (nt & 1) ? rx[rt][nt >> 1].w : rx[rt][nt >> 1].y;
                    x[rt][nt][0] = DT::to_f((u16)(lo & 0xffff)) + b.x; x[rt][nt][1] = DT::to_f((u16)(lo >> 16)) + b.y;
                    x[rt][nt][2] = DT::to_f((u16)(hi & 0xffff)) + b.z; x[rt][nt][3] = DT::to_f((u16)(hi >> 16)) + b.w;
                    asm("" : "+a"(x[rt][nt]));        // the accumulator lives in accumulation registers from here on
                    if ((nt & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {   // the tile's own loads: all issued, one wait the compiler can see (it does not know of the ring's transfers)
            uint2 rx[2][NT], rh[2][NT];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                int64_t row = row0 + 16 * rt + r16; row = row < a.rows ? row : a.rows - 1;
                const u16* xr = a.x + row * D; const u16* hr = a.h2 + row * D;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    rx[rt][nt] = *reinterpret_cast<const uint2*>(xr + 16 * nt + 4 * g);
                    rh[rt][nt] = *reinterpret_cast<const uint2*>(hr + 16 * nt + 4 * g);
                }
            }
            __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float4 b = *reinterpret_cast<const float4*>(B2 + 16 * nt + 4 * g);
                    x[rt][nt][0] = DT::to_f((u16)(rx[rt][nt].x & 0xffff)) + b.x; x[rt][nt][1] = DT::to_f((u16)(rx[rt][nt].x >> 16)) + b.y;
                    x[rt][nt][2] = DT::to_f((u16)(rx[rt][nt].y & 0xffff)) + b.z; x[rt][nt][3] = DT::to_f((u16)(rx[rt][nt].y >> 16)) + b.w;
                    hf[rt][nt >> 1].h[nt & 1] = rh[rt][nt];       // a lane's 4 features of tile nt are half of chunk nt / 2's operand fragment
                }
        }
        const int nch = a.F / 32;
        f32x4 acc[2][2];                                     // [tile of the chunk][row tile]
        auto up = [&](int ch) __attribute__((always_inline)) {
#pragma unroll
            for (int ntl = 0; ntl < 2; ++ntl) {
                const float4 b = *reinterpret_cast<const float4*>(B1 + 32 * ch + 16 * ntl + 4 * g);
                acc[ntl][0] = (f32x4){b.x, b.y, b.z, b.w}; acc[ntl][1] = acc[ntl][0];
            }
            static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                constexpr int half = decltype(j_)::value / 2, ntl = decltype(j_)::value % 2;
                sub(j_, [&](const s16x8 (&wf)[KB]) __attribute__((always_inline)) {
#pragma unroll
                    for (int ci = 0; ci < KB; ++ci)
#pragma unroll
                        for (int rt = 0; rt < 2; ++rt)
                            acc[ntl][rt] = DT::mfma32(wf[ci], hf[rt][half * KB + ci].v, acc[ntl][rt]);
                });
            });
        };
        // PIPE (one wave per SIMD: nothing else runs while a wave waits): the fragment reads run NBUF - 1 fragments ahead
        // of the MFMAs through a rotating set of NBUF registers quads, across stage boundaries too - before the two
        // MFMAs of fragment i are issued, fragment i + NBUF - 1 is requested (behind the next stage's admission when it
        // opens a stage), and a scheduling barrier keeps the request above the MFMAs.  SF is a multiple of NBUF, so a
        // fragment's register set is the same in every stage.
        constexpr bool PIPE = D == 384;
        constexpr int NBUF = 4, SF = G::SF;
        static_assert(!PIPE || SF % NBUF == 0, "rotating fragment registers");
        s16x8 wr[NBUF];
        // one stage: mm(i, fragment) per fragment; next: 0 = nothing follows in this tile, 1 = an odd stage (entered
        // without a barrier), 2 = an even one (the pair admission, which reuses the slot of the stage being left: every
        // wave's reads of it must have returned before the barrier)
        auto stage = [&](int next, auto&& mm) __attribute__((always_inline)) {
            static_for<0, SF>([&](auto i_) __attribute__((always_inline)) {
                constexpr int i = decltype(i_)::value, n = i + NBUF - 1;
                if constexpr (n < SF) wr[n % NBUF] = pipe.frag(n, lane);
                else if (next) {
                    if constexpr (n == SF) {
                        if (next == 2) { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); advance(Even{}); }
                        else advance(Odd{});
                    }
                    wr[n % NBUF] = pipe.frag(n - SF, lane);
                }
                __builtin_amdgcn_sched_barrier(0);
                mm(i_, wr[i % NBUF]);
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        // (wide: the stage's 32 columns in the paired order above - a lane's four of tile 0 and four of tile 1 adjacent)
        auto acc_init = [&](const float* bias, int ch, bool wide) __attribute__((always_inline)) {
#pragma unroll
            for (int ntl = 0; ntl < 2; ++ntl) {
                const float4 b = *reinterpret_cast<const float4*>(bias + 32 * ch + (wide ? 8 * g + 4 * ntl : 16 * ntl + 4 * g));
                acc[ntl][0] = (f32x4){b.x, b.y, b.z, b.w}; acc[ntl][1] = acc[ntl][0];
            }
        };
        auto up_init = [&](int ch) __attribute__((always_inline)) { acc_init(B1, ch, false); };
        auto up_mm = [&](auto i_, const s16x8& wf) __attribute__((always_inline)) {
            constexpr int j = decltype(i_)::value / KB, ci = decltype(i_)::value % KB, half = j / 2, ntl = j % 2;
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) acc[ntl][rt] = DT::mfma32(wf, hf[rt][half * KB + ci].v, acc[ntl][rt]);
        };
        advance(Even{});
        if constexpr (PIPE) {      // an odd stage follows W1(0): W1(1), or W2(0) when nch == 1
#pragma unroll
            for (int f = 0; f < NBUF - 1; ++f) wr[f] = pipe.frag(f, lane);
            if constexpr (PROJ && !LEAD) {
                // KC projection stages (even, odd, ...; KC is even, so W1(0) stays an even stage): stage c adds
                // Wo[:, 32 c .. 32 c + 31] times the attention output's chunk c into every feature tile
                static_for<0, KC>([&](auto c_) __attribute__((always_inline)) {
                    constexpr int c = decltype(c_)::value;
                    stage((c & 1) ? 2 : 1, [&](auto i_, const s16x8& wo) __attribute__((always_inline)) {
                        constexpr int i = decltype(i_)::value;
#pragma unroll
                        for (int rt = 0; rt < 2; ++rt) x[rt][i] = DT::mfma32(wo, hf[rt][c].v, x[rt][i]);
                    });
                });
                // W1(0) is admitted and its first fragments requested.  x1 rounded as the stream stores it, LayerNorm
                // on the rounded row (one pass, as the epilogue below), h2 rounded into the operand fragments, and the
                // FFN's accumulator x1 + b2
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    float s1 = 0.f, q1 = 0.f;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const uint32_t lo = bpack2<DT>(x[rt][nt][0], x[rt][nt][1]), hi = bpack2<DT>(x[rt][nt][2], x[rt][nt][3]);
                        f32x4 r;
                        r[0] = DT::to_f((u16)(lo & 0xffff)); r[1] = DT::to_f((u16)(lo >> 16));
                        r[2] = DT::to_f((u16)(hi & 0xffff)); r[3] = DT::to_f((u16)(hi >> 16));
#pragma unroll
                        for (int i = 0; i < 4; ++i) { s1 += r[i]; q1 = fmaf(r[i], r[i], q1); }
                        asm("" : "+a"(r));
                        x[rt][nt] = r;
                        if ((nt & 3) == 3) __builtin_amdgcn_sched_barrier(0);      // keeps the accumulator's trips through the vector registers short
                    }
                    rows_reduce2(s1, q1, OpAdd());
                    const float mean = s1 * (1.0f / D);
                    const float rstd = rsqrtf(fmaxf(fmaf(-mean, mean, q1 * (1.0f / D)), 0.f) + a.eps2);
                    const float shift = -mean * rstd;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const float4 gm = *reinterpret_cast<const float4*>(LN2G + foff(nt));
                        const float4 bt = *reinterpret_cast<const float4*>(LN2B + foff(nt));
                        const float4 b2 = *reinterpret_cast<const float4*>(B2 + foff(nt));
                        f32x4 r = x[rt][nt];
                        uint2 v;
                        v.x = bpack2<DT>(fmaf(fmaf(r[0], rstd, shift), gm.x, bt.x), fmaf(fmaf(r[1], rstd, shift), gm.y, bt.y));
                        v.y = bpack2<DT>(fmaf(fmaf(r[2], rstd, shift), gm.z, bt.z), fmaf(fmaf(r[3], rstd, shift), gm.w, bt.w));
                        hf[rt][nt >> 1].h[nt & 1] = v;
                        r[0] += b2.x; r[1] += b2.y; r[2] += b2.z; r[3] += b2.w;
                        asm("" : "+a"(r));
                        x[rt][nt] = r;
                        if ((nt & 1) == 1) __builtin_amdgcn_sched_barrier(0);      // (the scheduler would hoist every vector read above the first use)
                    }
                }
            }
            if constexpr (!LEAD) { up_init(0); stage(1, up_mm); }
        }
        else up(0);
        for (int ch = 0; ch < nch; ++ch) {
            BFrag8 hid[2];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    hid[rt].w[ntl * 2] = bpack2<DT>(apply_act16<ACT>(acc[ntl][rt][0]), apply_act16<ACT>(acc[ntl][rt][1]));
                    hid[rt].w[ntl * 2 + 1] = bpack2<DT>(apply_act16<ACT>(acc[ntl][rt][2]), apply_act16<ACT>(acc[ntl][rt][3]));
                }
            if (SAVE) {
                // the rounded hidden exactly as the down-projection consumes it: a lane holds 4 consecutive units of its
                // row per tile of the chunk (these stores sit in the vmcnt queue like any other: they can only make the
                // ring's admission waits stricter)
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    const int64_t row = row0 + 16 * rt + r16;
                    if (row < a.rows) {
                        u16* hr = a.hid + row * a.F + 32 * ch + 4 * g;
                        *reinterpret_cast<uint2*>(hr) = hid[rt].h[0];
                        *reinterpret_cast<uint2*>(hr + 16) = hid[rt].h[1];
                    }
                }
            }
            // stage parities: W1(0) even, then {W1(ch + 1) odd, W2(ch) even} ..., W2(last) odd
            if constexpr (PIPE) {
                // the stage in the ring and its first NBUF - 1 fragments were requested by the stage before
                if (ch + 1 < nch) { up_init(ch + 1); stage(2, up_mm); }                  // W1(ch + 1), then W2(ch): even
                // W2(ch); an odd stage follows but the last, which ends the tile or (PROJ with a projection behind) is followed by an even one
                stage(ch + 1 < nch ? 1 : (PROJ && a.nq > 0) ? 2 : 0, [&](auto i_, const s16x8& w2) __attribute__((always_inline)) {
                    constexpr int i = decltype(i_)::value;       // feature tile i
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt) x[rt][i] = DT::mfma32(w2, hid[rt].v, x[rt][i]);
                });
            } else {
                if (ch + 1 < nch) { advance(Odd{}); up(ch + 1); advance(Even{}); }
                else advance(Odd{});
                static_for<0, NSUB>([&](auto j_) __attribute__((always_inline)) {
                    constexpr int j = decltype(j_)::value;           // feature tiles [j * KB, +KB)
                    sub(j_, [&](const s16x8 (&w2)[KB]) __attribute__((always_inline)) {
#pragma unroll
                        for (int i = 0; i < KB; ++i)
#pragma unroll
                            for (int rt = 0; rt < 2; ++rt) x[rt][j * KB + i] = DT::mfma32(w2[i], hid[rt].v, x[rt][j * KB + i]);
                    });
                });
            }
        }
        // epilogue: round, store, optional LayerNorm on the rounded row
        float s[2] = {0.f, 0.f}, q[2] = {0.f, 0.f};
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int64_t row = row0 + 16 * rt + r16;
            u16* o = a.xo + row * D;
            uint2 vprev = make_uint2(0, 0);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                uint2 v;
                v.x = bpack2<DT>(x[rt][nt][0], x[rt][nt][1]); v.y = bpack2<DT>(x[rt][nt][2], x[rt][nt][3]);
                if constexpr (WIDE) {
                    if (nt & 1) { if (row < a.rows && !LEAD) *reinterpret_cast<uint4*>(o + 32 * (nt >> 1) + 8 * g) = make_uint4(vprev.x, vprev.y, v.x, v.y); }
                    else vprev = v;
                } else if (row < a.rows) *reinterpret_cast<uint2*>(o + 16 * nt + 4 * g) = v;
                if (LN) {
                    x[rt][nt][0] = DT::to_f((u16)(v.x & 0xffff)); x[rt][nt][1] = DT::to_f((u16)(v.x >> 16));
                    x[rt][nt][2] = DT::to_f((u16)(v.y & 0xffff)); x[rt][nt][3] = DT::to_f((u16)(v.y >> 16));
#pragma unroll
                    for (int i = 0; i < 4; ++i) { s[rt] += x[rt][nt][i]; q[rt] = fmaf(x[rt][nt][i], x[rt][nt][i], q[rt]); }
                }
            }
        }
        if (LN) {
            rows_reduce2(s[0], q[0], OpAdd());
            rows_reduce2(s[1], q[1], OpAdd());
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                const int64_t row = row0 + 16 * rt + r16;
                u16* o = a.ho + row * D;
                // one pass: var = E[x^2] - mean^2 clamped at 0 (python/beat_arena_env/csrc/layer_norm.cu:14-21)
                const float mean = s[rt] * (1.0f / D);
                const float rstd = rsqrtf(fmaxf(fmaf(-mean, mean, q[rt] * (1.0f / D)), 0.f) + a.eps);
                const float shift = -mean * rstd;
                uint2 hprev = make_uint2(0, 0);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float4 gm = *reinterpret_cast<const float4*>(LNG + foff(nt));
                    const float4 bt = *reinterpret_cast<const float4*>(LNB + foff(nt));
                    uint2 v;
                    v.x = bpack2<DT>(fmaf(fmaf(x[rt][nt][0], rstd, shift), gm.x, bt.x), fmaf(fmaf(x[rt][nt][1], rstd, shift), gm.y, bt.y));
                    v.y = bpack2<DT>(fmaf(fmaf(x[rt][nt][2], rstd, shift), gm.z, bt.z), fmaf(fmaf(x[rt][nt][3], rstd, shift), gm.w, bt.w));
                    if constexpr (WIDE) {
                        if (nt & 1) {
                            if (row < a.rows && (!PROJ || a.ho)) *reinterpret_cast<uint4*>(o + 32 * (nt >> 1) + 8 * g) = make_uint4(hprev.x, hprev.y, v.x, v.y);
                        } else hprev = v;
                    } else if (row < a.rows && (!PROJ || a.ho)) *reinterpret_cast<uint2*>(o + 16 * nt + 4 * g) = v;
                    if constexpr (PROJ) hf[rt][nt >> 1].h[nt & 1] = v;       // operand fragments of the projection behind
                }
            }
        }
        if constexpr (PROJ && LN) {
            // qo = ho Wn^T + bn: nq stages of 32 output columns in the up-projection's form (the first is admitted and its
            // first fragments are in flight), each stored as it completes
            const int ldq = 32 * a.nq;
            auto q_store = [&](int sq) __attribute__((always_inline)) {
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    const int64_t row = row0 + 16 * rt + r16;
                    if (row < a.rows) {       // the stage's columns in the paired order: 16 bytes per lane
                        uint4 v;
                        v.x = bpack2<DT>(acc[0][rt][0], acc[0][rt][1]); v.y = bpack2<DT>(acc[0][rt][2], acc[0][rt][3]);
                        v.z = bpack2<DT>(acc[1][rt][0], acc[1][rt][1]); v.w = bpack2<DT>(acc[1][rt][2], acc[1][rt][3]);
                        *reinterpret_cast<uint4*>(a.qo + row * ldq + 32 * sq + 8 * g) = v;
                    }
                }
            };
            for (int sq = 0; sq < a.nq; sq += 2) {       // nq is even: an even stage, then an odd one
                acc_init(BN, sq, true); stage(1, up_mm); q_store(sq);
                acc_init(BN, sq + 1, true); stage(sq + 2 < a.nq ? 2 : 0, up_mm); q_store(sq + 1);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // no transfer into LDS may outlive the workgroup
    blk_barrier();
}

struct FfnPackArgs { const u16* w0; const float* b0; const u16* w2; const float* b2; void* frags; float* vec; int F; };
// fragments of the 2 * F / 32 FFN stages from the 16-bit weights (a copy in fragment order, no rounding); one wave
// per fragment, one lane per 16-byte slot
template <int D>
__global__ __launch_bounds__(256) void ffn_pack_frags_kernel(FfnPackArgs a) {
    typedef Geo<D> G;
    constexpr int SF = G::SF;
    const int lane = threadIdx.x & 63, n16 = lane & 15, gg = lane >> 4;
    const int nch = a.F / 32;
    const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= 2 * nch * SF) return;
    const int s3 = f / SF, i = f % SF;
    bool upw; int ch;
    if (s3 == 0) { upw = true; ch = 0; }
    else if (s3 == 2 * nch - 1) { upw = false; ch = nch - 1; }
    else { upw = ((s3 - 1) & 1) == 0; ch = (s3 - 1) / 2 + (upw ? 1 : 0); }
    const u16* src; int ld, n, kbase = 0, c = 0;
    // d = 384 (the kernel's WIDE order): feature tiles' rows paired - A row m of tile i is feature
    // 32 (i / 2) + 8 (m / 4) + 4 (i % 2) + m % 4 -, and the k values of an INPUT-feature chunk in natural order
    constexpr bool WIDE = D == 384;
    if (upw) {
        const int burst = i / G::FB, rem = i % G::FB, ntl = rem / G::KB;
        c = burst * G::KB + rem % G::KB;
        src = a.w0; ld = D; n = 32 * ch + 16 * ntl + n16;
    } else { src = a.w2; ld = a.F; n = WIDE ? 32 * (i >> 1) + 8 * (n16 >> 2) + 4 * (i & 1) + (n16 & 3) : 16 * i + n16; kbase = 32 * ch; }
    u16 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[(int64_t)n * ld + kbase + (WIDE && upw ? 32 * c + 8 * gg + j : bperm_k(c, gg, j))];
    uint4 o;
    o.x = v[0] | ((uint32_t)v[1] << 16); o.y = v[2] | ((uint32_t)v[3] << 16);
    o.z = v[4] | ((uint32_t)v[5] << 16); o.w = v[6] | ((uint32_t)v[7] << 16);
    static_cast<uint4*>(a.frags)[(int64_t)f * 64 + lane] = o;
    if (f == 0) for (int k = lane; k < a.F + D; k += 64) a.vec[k] = k < a.F ? a.b0[k] : a.b2[k - a.F];
}

bool ffn_packed_shape_ok(int64_t d, int64_t F, int dtype) {
    if (d != 128 && d != 192 && d != 256 && d != 384) return false;
    if (F < 64 || F % 32 != 0 || F > 16384 || (dtype != BSRL_F16 && dtype != BSRL_BF16)) return false;
    const int slots = d == 128 ? 10 : d == 192 ? 7 : d == 256 ? 6 : 5;
    return 2 * (F / 32) >= slots;
}
int64_t ffn_frag_bytes(int64_t d, int64_t F) { return 2 * (F / 32) * (d / 16) * 1024; }
template <int D, int NW, int XS> size_t ffn_dyn_bytes(int F, bool proj = false, int nq = 0) {
    return (size_t)(((F + (proj ? 6 * D + 32 * nq : 3 * D)) / 4 + 63) & ~63) * 16 + (size_t)FfnRing<D, NW, XS>::SLOTS * FfnRing<D, NW, XS>::STAGE_BYTES;
}
template <typename DT, int D, int ACT, int NW, int XS = 0>
int ffn_launch_nw(const FfnArgs& a, bool ln, int cus, hipStream_t st) {
    const size_t dyn = ffn_dyn_bytes<D, NW, XS>(a.F);
    constexpr int WGS = ffn_wgs_per_cu<D, NW>();
    if (WGS * (dyn + 1024) > (size_t)LDS_BUDGET) return BSRL_UNSUPPORTED;
    const int64_t ntiles = (a.rows + NW * 32 - 1) / (NW * 32), slots = (int64_t)cus * WGS;
    const dim3 grid((unsigned)(ntiles < slots ? ntiles : slots));
    auto launch = [&](auto kern) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess)
            return (int)BSRL_UNSUPPORTED;
        hipLaunchKernelGGL(kern, grid, dim3(NW * 64), dyn, st, a);
        return (int)BSRL_OK;
    };
    if (a.hid) return ln ? launch(ffn_rows_kernel<DT, D, ACT, true, true, NW, XS>) : launch(ffn_rows_kernel<DT, D, ACT, false, true, NW, XS>);
    return ln ? launch(ffn_rows_kernel<DT, D, ACT, true, false, NW, XS>) : launch(ffn_rows_kernel<DT, D, ACT, false, false, NW, XS>);
}
template <typename DT, int D, int ACT>
int ffn_launch(const FfnArgs& a, bool ln, int cus, hipStream_t st) {
    if constexpr (D == 384) {
        // six slots of 24 KB where the vectors fit beside them (F up to 2560) and the image is that long, else five
        if (a.total_stages >= FfnRing<D, 4, 1>::SLOTS) {
            const int rc = ffn_launch_nw<DT, D, ACT, 4, 1>(a, ln, cus, st);
            if (rc != BSRL_UNSUPPORTED) return rc;
        }
        return ffn_launch_nw<DT, D, ACT, 4>(a, ln, cus, st);
    } else if constexpr (D != 256) {
        // two 4-wave workgroups per CU where two rings fit and the image is longer than the shorter ring
        if (a.total_stages >= FfnRing<D, 4>::SLOTS) {
            const int rc = ffn_launch_nw<DT, D, ACT, 4>(a, ln, cus, st);
            if (rc != BSRL_UNSUPPORTED) return rc;
        }
    }
    if constexpr (D != 384) return ffn_launch_nw<DT, D, ACT, 8>(a, ln, cus, st);
    return BSRL_UNSUPPORTED;
}

// the projection form (d = 384): six ring slots where the longer vector block leaves room, else five
template <typename DT, int ACT, int XS, bool LEAD = false>
int proj_ffn_launch_xs(const FfnArgs& a, bool ln, int cus, hipStream_t st) {
    constexpr int D = 384, NW = 4;
    const size_t dyn = ffn_dyn_bytes<D, NW, XS>(a.F, true, a.nq);
    if (dyn + 1024 > (size_t)LDS_BUDGET || a.total_stages < FfnRing<D, NW, XS>::SLOTS) return BSRL_UNSUPPORTED;
    const int64_t ntiles = (a.rows + NW * 32 - 1) / (NW * 32);
    const dim3 grid((unsigned)(ntiles < cus ? ntiles : cus));
    auto launch = [&](auto kern) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess)
            return (int)BSRL_UNSUPPORTED;
        hipLaunchKernelGGL(kern, grid, dim3(NW * 64), dyn, st, a);
        return (int)BSRL_OK;
    };
    if constexpr (LEAD) return launch(ffn_rows_kernel<DT, D, ACT, true, false, NW, XS, true, true>);
    else return ln ? launch(ffn_rows_kernel<DT, D, ACT, true, false, NW, XS, true>) : launch(ffn_rows_kernel<DT, D, ACT, false, false, NW, XS, true>);
}
template <typename DT, int ACT>
int proj_ffn_launch(const FfnArgs& a, bool ln, int cus, hipStream_t st) {
    const int rc = proj_ffn_launch_xs<DT, ACT, 1>(a, ln, cus, st);
    return rc != BSRL_UNSUPPORTED ? rc : proj_ffn_launch_xs<DT, ACT, 0>(a, ln, cus, st);
}

struct ProjPackArgs { const u16* wo; const float* bo; void* frags; float* vec_bo; const u16* wn; const float* bn; void* nfrags; int nq; };
// the d / 32 output-projection stages in front of the FFN stages: stage c, fragment i = rows [16 i, +16) of Wo, columns
// [32 c, +32) in the operand order of a hidden chunk (the form of a W2 stage); one wave per fragment
template <int D>
__global__ __launch_bounds__(256) void proj_pack_frags_kernel(ProjPackArgs a) {
    constexpr int SF = Geo<D>::SF, KC = Geo<D>::KC;
    const int lane = threadIdx.x & 63, n16 = lane & 15, gg = lane >> 4;
    const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= KC * SF) return;
    const int c = f / SF, i = f % SF;
    u16 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)       // rows in the paired order, the attention output's k values in natural order
        v[j] = a.wo[(int64_t)(32 * (i >> 1) + 8 * (n16 >> 2) + 4 * (i & 1) + (n16 & 3)) * D + 32 * c + 8 * gg + j];
    uint4 o;
    o.x = v[0] | ((uint32_t)v[1] << 16); o.y = v[2] | ((uint32_t)v[3] << 16);
    o.z = v[4] | ((uint32_t)v[5] << 16); o.w = v[6] | ((uint32_t)v[7] << 16);
    static_cast<uint4*>(a.frags)[(int64_t)f * 64 + lane] = o;
    if (f == 0) for (int k = lane; k < D; k += 64) a.vec_bo[k] = a.bo[k];
}
// the nq stages of the projection behind the FFN: stage s = rows [32 s, +32) of Wn in the form of a W1 stage
template <int D>
__global__ __launch_bounds__(256) void next_pack_frags_kernel(ProjPackArgs a) {
    typedef Geo<D> G;
    constexpr int SF = G::SF;
    const int lane = threadIdx.x & 63, n16 = lane & 15, gg = lane >> 4;
    const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= a.nq * SF) return;
    const int sq = f / SF, i = f % SF;
    const int burst = i / G::FB, rem = i % G::FB, ntl = rem / G::KB, c = burst * G::KB + rem % G::KB;
    u16 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)       // the stage's 32 columns in the paired order, k natural
        v[j] = a.wn[(int64_t)(32 * sq + 8 * (n16 >> 2) + 4 * ntl + (n16 & 3)) * D + 32 * c + 8 * gg + j];
    uint4 o;
    o.x = v[0] | ((uint32_t)v[1] << 16); o.y = v[2] | ((uint32_t)v[3] << 16);
    o.z = v[4] | ((uint32_t)v[5] << 16); o.w = v[6] | ((uint32_t)v[7] << 16);
    static_cast<uint4*>(a.nfrags)[(int64_t)f * 64 + lane] = o;
    if (f == 0) for (int k = lane; k < 32 * a.nq; k += 64) a.vec_bo[D + k] = a.bn[k];
    // an image without the stages in front (no output projection): the kernel's b2 | bo are zeros
    if (f == 0 && a.wo == nullptr) for (int k = lane; k < 2 * D; k += 64) a.vec_bo[k - D] = 0.f;
}
bool proj_ffn_shape_ok(int64_t d, int64_t F, int64_t n_next, int dtype) {
    if (!(d == 384 && ffn_packed_shape_ok(d, F, dtype) && n_next >= 0 && n_next % 64 == 0 && n_next <= 3 * d)) return false;
    // the vectors (b0, b2, three LayerNorm pairs' worth, bo, bn) must fit LDS beside the five-slot ring
    return (size_t)(F + 6 * d + n_next) * 4 + 1024 + 5 * FfnRing<384, 4, 0>::STAGE_BYTES + 1024 <= (size_t)LDS_BUDGET;
}
int64_t proj_frag_bytes(int64_t d) { return (d / 32) * (d / 16) * 1024; }

}  // namespace

extern "C" int64_t bsrl_proj_ffn_pack_size(int64_t d, int64_t F, int64_t n_next, int dtype) {
    if (!proj_ffn_shape_ok(d, F, n_next, dtype)) return 0;
    return proj_frag_bytes(d) + ffn_frag_bytes(d, F) + (n_next / 32) * (d / 16) * 1024 + (F + 2 * d + n_next) * 4;
}

extern "C" int bsrl_proj_ffn_pack(const void* wo, const float* bo, const void* w0, const float* b0, const void* w2,
                                  const float* b2, const void* wn, const float* bn, int64_t n_next, int64_t d, int64_t F,
                                  int dtype, void* image, bsrl_stream stream) {
    if (!wo || !bo || !w0 || !b0 || !w2 || !b2 || !image) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_pack: null pointer");
    if (!proj_ffn_shape_ok(d, F, n_next, dtype)) return BSRL_UNSUPPORTED;
    if (n_next > 0 && (!wn || !bn)) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_pack: n_next > 0 needs wn and bn");
    if (!bsrl_aligned(image, 16)) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_pack: image must be 16-byte aligned");
    char* img = static_cast<char*>(image);
    char* ffn_frags = img + proj_frag_bytes(d);
    char* next_frags = ffn_frags + ffn_frag_bytes(d, F);
    float* vec = reinterpret_cast<float*>(next_frags + (n_next / 32) * (d / 16) * 1024);      // b0 (F) | b2 (d) | bo (d) | bn (n_next)
    hipStream_t st = static_cast<hipStream_t>(stream);
    ProjPackArgs pp{static_cast<const u16*>(wo), bo, image, vec + F + d, static_cast<const u16*>(wn), bn, next_frags, (int)(n_next / 32)};
    const int64_t npf = (d / 32) * (d / 16);
    hipLaunchKernelGGL(proj_pack_frags_kernel<384>, dim3((unsigned)((npf + 3) / 4)), dim3(256), 0, st, pp);
    if (n_next > 0) {
        const int64_t nnf = (n_next / 32) * (d / 16);
        hipLaunchKernelGGL(next_pack_frags_kernel<384>, dim3((unsigned)((nnf + 3) / 4)), dim3(256), 0, st, pp);
    }
    FfnPackArgs pa{static_cast<const u16*>(w0), b0, static_cast<const u16*>(w2), b2, ffn_frags, vec, (int)F};
    const int64_t nfrags = 2 * (F / 32) * (d / 16);
    hipLaunchKernelGGL(ffn_pack_frags_kernel<384>, dim3((unsigned)((nfrags + 3) / 4)), dim3(256), 0, st, pa);
    BSRL_CHECK_LAUNCH("bsrl_proj_ffn_pack");
    return BSRL_OK;
}

extern "C" int bsrl_proj_ffn_packed(const void* image, const void* att, const void* x, const float* ln2_w, const float* ln2_b,
                                    float eps2, const float* ln_w, const float* ln_b, float eps, void* xo, void* ho,
                                    void* qo, int64_t n_next, int64_t rows, int64_t d, int64_t F, int act, int dtype,
                                    bsrl_stream stream) {
    if (!image || !att || !x || !xo || !ln2_w || !ln2_b) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: null pointer");
    if ((ln_w == nullptr) != (ln_b == nullptr)) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: ln_w and ln_b go together");
    if (n_next == 0 && (ln_w == nullptr) != (ho == nullptr))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: without a projection behind, ln_w / ln_b and ho go together");
    if (n_next > 0 && (!ln_w || !qo)) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: n_next > 0 needs ln_w, ln_b and qo");
    if (ho && !ln_w) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: ho needs ln_w and ln_b");
    if (!proj_ffn_shape_ok(d, F, n_next, dtype) || (act != BSRL_ACT_RELU && act != BSRL_ACT_GELU)) return BSRL_UNSUPPORTED;
    if (rows < 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: rows < 0");
    if (!bsrl_aligned(image, 16) || !bsrl_aligned(x, 8) || !bsrl_aligned(att, 8) || !bsrl_aligned(xo, 8) || (ho && !bsrl_aligned(ho, 8)) ||
        (qo && !bsrl_aligned(qo, 8)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: image must be 16-byte, rows 8-byte aligned");
    if (!bsrl_aligned(x, 16) || !bsrl_aligned(att, 16) || !bsrl_aligned(xo, 16) || (ho && !bsrl_aligned(ho, 16)) || (qo && !bsrl_aligned(qo, 16)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_proj_ffn_packed: rows must be 16-byte aligned");
    if (rows == 0) return BSRL_OK;
    FfnArgs a;
    a.frags = static_cast<const uint2*>(image);
    a.vec = reinterpret_cast<const float*>(static_cast<const char*>(image) + proj_frag_bytes(d) + ffn_frag_bytes(d, F) +
                                           (n_next / 32) * (d / 16) * 1024);
    a.x = static_cast<const u16*>(x); a.h2 = static_cast<const u16*>(att);
    a.xo = static_cast<u16*>(xo); a.ho = static_cast<u16*>(ho); a.hid = nullptr;
    a.ln_w = ln_w; a.ln_b = ln_b; a.eps = eps; a.rows = rows; a.F = (int)F;
    a.total_stages = (int)(d / 32 + 2 * (F / 32) + n_next / 32);
    a.ln2_w = ln2_w; a.ln2_b = ln2_b; a.eps2 = eps2;
    a.qo = static_cast<u16*>(qo); a.nq = (int)(n_next / 32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    const bool relu = act == BSRL_ACT_RELU, ln = ln_w != nullptr;
    int rc;
    if (dtype == BSRL_F16) rc = relu ? proj_ffn_launch<F16, BSRL_ACT_RELU>(a, ln, cus, st) : proj_ffn_launch<F16, BSRL_ACT_GELU>(a, ln, cus, st);
    else rc = relu ? proj_ffn_launch<BF16, BSRL_ACT_RELU>(a, ln, cus, st) : proj_ffn_launch<BF16, BSRL_ACT_GELU>(a, ln, cus, st);
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH("bsrl_proj_ffn_packed");
    return BSRL_OK;
}

// LayerNorm + packed projection alone: the block-tail kernel with nothing in front of its last phase
namespace {
bool ln_proj_shape_ok(int64_t d, int64_t n_next, int dtype) {
    return d == 384 && (dtype == BSRL_F16 || dtype == BSRL_BF16) && n_next >= 6 * 32 && n_next % 64 == 0 && n_next <= 3 * d;
}
}  // namespace

extern "C" int64_t bsrl_ln_proj_pack_size(int64_t d, int64_t n_next, int dtype) {
    if (!ln_proj_shape_ok(d, n_next, dtype)) return 0;
    return (n_next / 32) * (d / 16) * 1024 + (2 * d + n_next) * 4;
}

extern "C" int bsrl_ln_proj_pack(const void* wn, const float* bn, int64_t n_next, int64_t d, int dtype, void* image,
                                 bsrl_stream stream) {
    if (!wn || !bn || !image) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_proj_pack: null pointer");
    if (!ln_proj_shape_ok(d, n_next, dtype)) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(image, 16)) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_proj_pack: image must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    float* vec = reinterpret_cast<float*>(static_cast<char*>(image) + (n_next / 32) * (d / 16) * 1024);   // zeros (2 d: the kernel's b2 | bo) | bn
    ProjPackArgs pp{nullptr, nullptr, nullptr, vec + d, static_cast<const u16*>(wn), bn, image, (int)(n_next / 32)};
    const int64_t nnf = (n_next / 32) * (d / 16);
    hipLaunchKernelGGL(next_pack_frags_kernel<384>, dim3((unsigned)((nnf + 3) / 4)), dim3(256), 0, st, pp);
    BSRL_CHECK_LAUNCH("bsrl_ln_proj_pack");
    return BSRL_OK;
}

extern "C" int bsrl_ln_proj_packed(const void* image, const void* x, const float* ln_w, const float* ln_b, float eps,
                                   void* ho, void* qo, int64_t n_next, int64_t rows, int64_t d, int dtype, bsrl_stream stream) {
    if (!image || !x || !ln_w || !ln_b || !qo) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_proj_packed: null pointer");
    if (!ln_proj_shape_ok(d, n_next, dtype)) return BSRL_UNSUPPORTED;
    if (rows < 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_proj_packed: rows < 0");
    if (!bsrl_aligned(image, 16) || !bsrl_aligned(x, 16) || (ho && !bsrl_aligned(ho, 16)) || !bsrl_aligned(qo, 16))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ln_proj_packed: image and rows must be 16-byte aligned");
    if (rows == 0) return BSRL_OK;
    FfnArgs a;
    a.frags = static_cast<const uint2*>(image);
    a.vec = reinterpret_cast<const float*>(static_cast<const char*>(image) + (n_next / 32) * (d / 16) * 1024);
    a.x = static_cast<const u16*>(x); a.h2 = a.x;
    a.xo = nullptr; a.ho = static_cast<u16*>(ho); a.hid = nullptr;
    a.ln_w = ln_w; a.ln_b = ln_b; a.eps = eps; a.rows = rows; a.F = 0;
    a.total_stages = (int)(n_next / 32);
    a.ln2_w = ln_w; a.ln2_b = ln_b; a.eps2 = eps;
    a.qo = static_cast<u16*>(qo); a.nq = (int)(n_next / 32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    int rc = dtype == BSRL_F16 ? proj_ffn_launch_xs<F16, BSRL_ACT_RELU, 1, true>(a, true, cus, st)
                               : proj_ffn_launch_xs<BF16, BSRL_ACT_RELU, 1, true>(a, true, cus, st);
    if (rc == BSRL_UNSUPPORTED)
        rc = dtype == BSRL_F16 ? proj_ffn_launch_xs<F16, BSRL_ACT_RELU, 0, true>(a, true, cus, st)
                               : proj_ffn_launch_xs<BF16, BSRL_ACT_RELU, 0, true>(a, true, cus, st);
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH("bsrl_ln_proj_packed");
    return BSRL_OK;
}

extern "C" int64_t bsrl_ffn_pack_size(int64_t d, int64_t F, int dtype) {
    if (!ffn_packed_shape_ok(d, F, dtype)) return 0;
    return ffn_frag_bytes(d, F) + (F + d) * 4;
}

extern "C" int bsrl_ffn_pack(const void* w0, const float* b0, const void* w2, const float* b2, int64_t d, int64_t F,
                             int dtype, void* image, bsrl_stream stream) {
    if (!w0 || !b0 || !w2 || !b2 || !image) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_pack: null pointer");
    if (!ffn_packed_shape_ok(d, F, dtype)) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(image, 16)) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_pack: image must be 16-byte aligned");
    FfnPackArgs pa{static_cast<const u16*>(w0), b0, static_cast<const u16*>(w2), b2, image,
                   reinterpret_cast<float*>(static_cast<char*>(image) + ffn_frag_bytes(d, F)), (int)F};
    const int64_t nfrags = 2 * (F / 32) * (d / 16);
    const dim3 grid((unsigned)((nfrags + 3) / 4));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (d == 128) hipLaunchKernelGGL(ffn_pack_frags_kernel<128>, grid, dim3(256), 0, st, pa);
    else if (d == 192) hipLaunchKernelGGL(ffn_pack_frags_kernel<192>, grid, dim3(256), 0, st, pa);
    else if (d == 256) hipLaunchKernelGGL(ffn_pack_frags_kernel<256>, grid, dim3(256), 0, st, pa);
    else hipLaunchKernelGGL(ffn_pack_frags_kernel<384>, grid, dim3(256), 0, st, pa);
    BSRL_CHECK_LAUNCH("bsrl_ffn_pack");
    return BSRL_OK;
}

extern "C" int bsrl_ffn_packed(const void* image, const void* x, const void* h2, const float* ln_w, const float* ln_b,
                               float eps, void* xo, void* ho, void* hid, int64_t rows, int64_t d, int64_t F, int act,
                               int dtype, bsrl_stream stream) {
    if (!image || !x || !h2 || !xo) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_packed: null pointer");
    if ((ln_w == nullptr) != (ho == nullptr) || (ln_w == nullptr) != (ln_b == nullptr))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_packed: ln_w, ln_b and ho go together");
    if (!ffn_packed_shape_ok(d, F, dtype) || (act != BSRL_ACT_RELU && act != BSRL_ACT_GELU)) return BSRL_UNSUPPORTED;
    if (rows < 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_packed: rows < 0");
    if (!bsrl_aligned(image, 16) || !bsrl_aligned(x, 8) || !bsrl_aligned(h2, 8) || !bsrl_aligned(xo, 8) || (ho && !bsrl_aligned(ho, 8)) ||
        (hid && !bsrl_aligned(hid, 8)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_packed: image must be 16-byte, rows 8-byte aligned");
    if (d == 384 && (!bsrl_aligned(x, 16) || !bsrl_aligned(h2, 16) || !bsrl_aligned(xo, 16) || (ho && !bsrl_aligned(ho, 16))))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_ffn_packed: at d = 384 rows must be 16-byte aligned (they move in 16-byte pieces)");
    if (rows == 0) return BSRL_OK;
    FfnArgs a;
    a.frags = static_cast<const uint2*>(image);
    a.vec = reinterpret_cast<const float*>(static_cast<const char*>(image) + ffn_frag_bytes(d, F));
    a.x = static_cast<const u16*>(x); a.h2 = static_cast<const u16*>(h2);
    a.xo = static_cast<u16*>(xo); a.ho = static_cast<u16*>(ho); a.hid = static_cast<u16*>(hid);
    a.ln_w = ln_w; a.ln_b = ln_b; a.eps = eps; a.rows = rows; a.F = (int)F; a.total_stages = (int)(2 * (F / 32));
    a.ln2_w = a.ln2_b = nullptr; a.eps2 = 0.f; a.qo = nullptr; a.nq = 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    const bool relu = act == BSRL_ACT_RELU, f16 = dtype == BSRL_F16, ln = ln_w != nullptr;
    int rc;
    if (d == 128) {
        if (f16) rc = relu ? ffn_launch<F16, 128, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<F16, 128, BSRL_ACT_GELU>(a, ln, cus, st);
        else rc = relu ? ffn_launch<BF16, 128, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<BF16, 128, BSRL_ACT_GELU>(a, ln, cus, st);
    } else if (d == 192) {
        if (f16) rc = relu ? ffn_launch<F16, 192, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<F16, 192, BSRL_ACT_GELU>(a, ln, cus, st);
        else rc = relu ? ffn_launch<BF16, 192, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<BF16, 192, BSRL_ACT_GELU>(a, ln, cus, st);
    } else if (d == 256) {
        if (f16) rc = relu ? ffn_launch<F16, 256, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<F16, 256, BSRL_ACT_GELU>(a, ln, cus, st);
        else rc = relu ? ffn_launch<BF16, 256, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<BF16, 256, BSRL_ACT_GELU>(a, ln, cus, st);
    } else {
        if (f16) rc = relu ? ffn_launch<F16, 384, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<F16, 384, BSRL_ACT_GELU>(a, ln, cus, st);
        else rc = relu ? ffn_launch<BF16, 384, BSRL_ACT_RELU>(a, ln, cus, st) : ffn_launch<BF16, 384, BSRL_ACT_GELU>(a, ln, cus, st);
    }
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH("bsrl_ffn_packed");
    return BSRL_OK;
}

extern "C" int64_t bsrl_blocks_pack_size(const bsrl_blocks_desc* d) {
    if (!blocks_shape_ok(d)) return 0;
    return blocks_frag_bytes(d) + (int64_t)d->n_layers * (9 * d->d + d->ffn) * 4;
}

extern "C" int bsrl_blocks_pack(const bsrl_blocks_desc* d, const bsrl_blocks_params* p, void* packed, bsrl_stream stream) {
    if (!d || !p || !packed) BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_pack: null pointer");
    if (!blocks_shape_ok(d)) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(packed, 16)) BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_pack: image must be 16-byte aligned");
    for (int l = 0; l < d->n_layers; ++l) {
        const float* const* ptrs = reinterpret_cast<const float* const*>(&p->blk[l]);
        for (int i = 0; i < 16; ++i)
            if (!ptrs[i]) BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_pack: null parameter pointer in block %d", l);
    }
    BlkPackArgs pa;
    pa.p = *p; pa.frags = packed;
    pa.vec = reinterpret_cast<float*>(static_cast<char*>(packed) + blocks_frag_bytes(d));
    pa.n_layers = d->n_layers; pa.F = d->ffn;
    const int64_t nfrags = blocks_stages(d) * (d->d / 16);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (d->d == 128) { if (d->dtype == BSRL_F16) pack_launch<F16, 128, 32>(pa, nfrags, st); else pack_launch<BF16, 128, 32>(pa, nfrags, st); }
    else if (d->d == 256) { if (d->dtype == BSRL_F16) pack_launch<F16, 256, 32>(pa, nfrags, st); else pack_launch<BF16, 256, 32>(pa, nfrags, st); }
    else { if (d->dtype == BSRL_F16) pack_launch<F16, 192, 48>(pa, nfrags, st); else pack_launch<BF16, 192, 48>(pa, nfrags, st); }
    BSRL_CHECK_LAUNCH("bsrl_blocks_pack");
    return BSRL_OK;
}

extern "C" int bsrl_blocks_forward(const bsrl_blocks_desc* d, const void* packed, const void* x_in, const void* key_bias,
                                   void* x_res, void* x_out, int64_t B, bsrl_stream stream) {
    if (!d || !packed || !x_in || !key_bias || !x_out) BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_forward: null pointer");
    if (!blocks_shape_ok(d)) return BSRL_UNSUPPORTED;
    if (B < 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_forward: B < 0");
    if (!bsrl_aligned(packed, 16) || !bsrl_aligned(x_in, 8) || !bsrl_aligned(x_out, 8) || (x_res && !bsrl_aligned(x_res, 8)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_blocks_forward: image must be 16-byte, token streams 8-byte aligned");
    if (B == 0) return BSRL_OK;
    BlkArgs a;
    a.frags = static_cast<const uint2*>(packed);
    a.vec = reinterpret_cast<const float*>(static_cast<const char*>(packed) + blocks_frag_bytes(d));
    a.x_in = static_cast<const u16*>(x_in); a.key_bias = static_cast<const u16*>(key_bias);
    a.x_res = static_cast<u16*>(x_res); a.x_out = static_cast<u16*>(x_out);
    a.B = B; a.n_layers = d->n_layers; a.F = d->ffn; a.T = d->T; a.n_queries = d->n_queries;
    a.total_stages = (int)blocks_stages(d);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    int rc;
    const bool relu = d->act == BSRL_ACT_RELU, f16 = d->dtype == BSRL_F16;
    if (d->d == 128) {
        if (f16) rc = relu ? fwd_launch<F16, 128, 32, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<F16, 128, 32, BSRL_ACT_GELU>(a, cus, st);
        else rc = relu ? fwd_launch<BF16, 128, 32, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<BF16, 128, 32, BSRL_ACT_GELU>(a, cus, st);
    } else if (d->d == 256) {
        if (f16) rc = relu ? fwd_launch<F16, 256, 32, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<F16, 256, 32, BSRL_ACT_GELU>(a, cus, st);
        else rc = relu ? fwd_launch<BF16, 256, 32, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<BF16, 256, 32, BSRL_ACT_GELU>(a, cus, st);
    } else {
        if (f16) rc = relu ? fwd_launch<F16, 192, 48, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<F16, 192, 48, BSRL_ACT_GELU>(a, cus, st);
        else rc = relu ? fwd_launch<BF16, 192, 48, BSRL_ACT_RELU>(a, cus, st) : fwd_launch<BF16, 192, 48, BSRL_ACT_GELU>(a, cus, st);
    }
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH("bsrl_blocks_forward");
    return BSRL_OK;
}
