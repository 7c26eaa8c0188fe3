// Weight-resident streaming linear for many rows and a modest K: y = act(x W^T + b) (+ residual) (* ReLU gate).
//
// The policy's token-level Linears have millions of rows and K = 128 .. 256 on their input side, i.e. they are
// HBM streams (x in, y out) with a small weight.  (At larger K the resident block shrinks to a few 16-feature tiles
// and x would be re-read once per column block: those shapes stay on the LDS-tiled kernel.)  This kernel keeps a block of the weight - MT 16-feature tiles x all
// of K - resident in LDS in MFMA fragment order for the whole life of a persistent workgroup, and every
// wave streams its own 32-row tiles of x: whole rows, consecutive lanes on consecutive 16-byte pieces, one tile
// ahead of the MFMAs, turned into B fragments through a small per-wave LDS tile.  (Loading the fragments straight
// from global memory - lane = row, the 4 lanes of a row 16 lanes apart - touches 16 rows x 64 B per wave
// instruction: with everything but the loads cut out the kernel read at 3.65 TB/s that way and reads at 4.8 TB/s
// with whole-row loads; a plain 16-byte-per-lane read reaches 6.3 TB/s on this part.)  The register arrays
// that live across the tile loop are native vector types: arrays of HIP's uint4 class stayed in scratch.  There is
// no workgroup barrier after the prologue, so the 8 waves of a workgroup drift freely and hide each other's
// memory latency.
// Per 32-k chunk a wave reads MT fragments (1 KB each) from LDS for 2 MT MFMAs (two 16-row tiles share
// each fragment): the LDS read path allows ~50 % of MFMA peak, which is above what the HBM stream needs
// at these K.  Bias, activation, residual and gate are applied in registers (a lane holds 4 consecutive
// features of one row); the rounded results of 16 rows then cross a per-wave LDS tile so that they leave as
// 16-byte stores covering whole row segments - written as 32-byte pieces straight from the MFMA layout the
// same kernel ran at 3.1 TB/s instead of the 5 TB/s a plain copy reaches on this part (measured: the stores
// alone cost as much as the whole read stream).
// Column blocks of the same rows are mapped to the same XCD (block id % 8) and walk the rows in the same
// order, so x is fetched from HBM once and re-read from that XCD's L2 by the other column blocks.
//
// Same arithmetic contract as the other linear kernels (fp32 accumulate in a fixed k order, a row's
// result independent of the batch); the entry point picks by shape.
#include "linear_args.h"

namespace {

constexpr int ST_THREADS = 512;                  // 8 waves share one resident weight block
constexpr int ST_ROWS = 32;                      // rows per wave tile (2 MFMA row tiles)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ACT and AUX (0 none, 1 residual, 2 ReLU gate) are compile-time: with run-time switches the epilogue was 2270 VALU
// instructions and 248 branches per 32-row tile and took 12k of a tile's 18.5k cycles (traced with s_memtime), twice
// what its 144 MFMAs took.
template <typename DT, int KC, int MT, int ACT, int AUX>
__global__ __launch_bounds__(ST_THREADS) void linear_stream_kernel(LinArgs a, int nb, int walkers) {
    extern __shared__ __attribute__((aligned(16))) uint4 wl[];           // [MT * KC][64] fragments, MT * 16 bias floats, 8 wave tiles
    constexpr int KE = KC * 32;                                           // K
    constexpr int TP = (KE > MT * 16 ? KE : MT * 16) + 8;                 // wave tile row pitch (elements): rows 16 B off a bank period
    constexpr int PPR = KE / 8;                                           // 16-byte pieces per x row
    constexpr int NLD = (16 * PPR + WAVE - 1) / WAVE;                     // pieces per lane for 16 rows of x
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    // block id -> (walker, column block): the nb column blocks of one walker share id % 8, i.e. one XCD
    const int b = blockIdx.x;
    const int cb = (b >> 3) % nb;
    const int walker = ((b >> 3) / nb) * 8 + (b & 7);
    if (walker >= walkers) return;
    const int m0 = cb * MT * 16;
    const u16* w = static_cast<const u16*>(a.w);
    // resident weight block: fragment (mt, kc), lane l <- W[m0 + 16 mt + l % 16][32 kc + 8 (l / 16) .. + 7]
    // every load of the block is issued before the first LDS write: one memory round trip for the prologue, not one
    // per pass (with few rows per workgroup the prologue is most of the kernel)
    constexpr int WPASS = (MT * KC * 64 + ST_THREADS - 1) / ST_THREADS;
    u32x4 wv[WPASS];
#pragma unroll
    for (int it = 0; it < WPASS; ++it) {
        const int i = it * ST_THREADS + tid;
        const int l = i & 63, f = i >> 6, mt = f / KC, kc = f % KC;
        const int m = m0 + mt * 16 + (l & 15);
        wv[it] = (u32x4){0u, 0u, 0u, 0u};
        if (i < MT * KC * 64 && m < a.M) wv[it] = *reinterpret_cast<const u32x4*>(w + (int64_t)m * KE + kc * 32 + 8 * (l >> 4));
    }
#pragma unroll
    for (int it = 0; it < WPASS; ++it) {
        const int i = it * ST_THREADS + tid;
        if (i < MT * KC * 64) wl[i] = __builtin_bit_cast(uint4, wv[it]);
    }
    float* bl = reinterpret_cast<float*>(wl + MT * KC * 64);
    u16* wt = reinterpret_cast<u16*>(bl + MT * 16) + wave * (16 * TP);   // this wave's 16-row tile: x on the way in, y on the way out
    for (int i = tid; i < MT * 16; i += ST_THREADS) bl[i] = (a.bias && m0 + i < a.M) ? a.bias[m0 + i] : 0.f;
    __syncthreads();                                                      // the only barrier: waves are on their own from here

    const u16* x = static_cast<const u16*>(a.x);
    const int64_t ntiles = (a.rows + ST_ROWS - 1) / ST_ROWS;
    const int64_t stride = (int64_t)walkers * 8;
    int64_t tile = (int64_t)walker * 8 + wave;
    if (tile >= ntiles) return;
    // x arrives as whole rows: consecutive lanes load consecutive 16-byte pieces (a wave instruction = 1 KB of
    // contiguous memory when rows are dense), one 32-row tile ahead of the MFMAs
    u32x4 pa[NLD], pb[NLD];                                               // rows 0..15 and 16..31 of the tile in flight
#define ST_FETCH(t)                                                                                                   \
    _Pragma("unroll") for (int it = 0; it < NLD; ++it) {                                                               \
        const int p = it * WAVE + lane, r = p / PPR, part = p % PPR;                                                  \
        int64_t ra = (t) * ST_ROWS + r, rb = ra + 16;                                                                 \
        ra = ra < a.rows ? ra : a.rows - 1;                                                                           \
        rb = rb < a.rows ? rb : a.rows - 1;                                                                           \
        pa[it] = *reinterpret_cast<const u32x4*>(x + ra * a.ldx + part * 8);                                          \
        pb[it] = *reinterpret_cast<const u32x4*>(x + rb * a.ldx + part * 8);                                          \
    }
    ST_FETCH(tile)
    const u16* res = static_cast<const u16*>(a.res);
    const u16* gate = static_cast<const u16*>(a.gate);
    u16* y = static_cast<u16*>(a.y);
    for (; tile < ntiles; tile += stride) {
        // rows -> B fragments through the wave tile: lane (r16, g) of chunk kc holds x[16 h + r16][32 kc + 8 g .. + 7]
        u32x4 xf0[KC], xf1[KC];
#pragma unroll
        for (int it = 0; it < NLD; ++it) {
            const int p = it * WAVE + lane;
            if (NLD * WAVE == 16 * PPR || p < 16 * PPR) *reinterpret_cast<u32x4*>(wt + (p / PPR) * TP + (p % PPR) * 8) = pa[it];
        }
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) xf0[kc] = *reinterpret_cast<const u32x4*>(wt + r16 * TP + kc * 32 + 8 * g);
#pragma unroll
        for (int it = 0; it < NLD; ++it) {
            const int p = it * WAVE + lane;
            if (NLD * WAVE == 16 * PPR || p < 16 * PPR) *reinterpret_cast<u32x4*>(wt + (p / PPR) * TP + (p % PPR) * 8) = pb[it];
        }
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) xf1[kc] = *reinterpret_cast<const u32x4*>(wt + r16 * TP + kc * 32 + 8 * g);
        ST_FETCH(tile + stride)                                         // rows past the end clamp to the last row: always a valid load
        f32x4 acc[MT][2];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) { acc[mt][0] = (f32x4){0.f, 0.f, 0.f, 0.f}; acc[mt][1] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const s16x8 x0 = __builtin_bit_cast(s16x8, xf0[kc]), x1 = __builtin_bit_cast(s16x8, xf1[kc]);
            // fragments are read a pair ahead of their MFMAs and no further: without the pins the scheduler hoists
            // every LDS read of the tile to the top and spills the accumulators
#pragma unroll
            for (int mt = 0; mt < MT; mt += 2) {
                const s16x8 wf0 = __builtin_bit_cast(s16x8, wl[(mt * KC + kc) * 64 + lane]);
                const s16x8 wf1 = __builtin_bit_cast(s16x8, wl[((mt + 1) * KC + kc) * 64 + lane]);
                acc[mt][0] = DT::mfma32(wf0, x0, acc[mt][0]);
                acc[mt][1] = DT::mfma32(wf0, x1, acc[mt][1]);
                acc[mt + 1][0] = DT::mfma32(wf1, x0, acc[mt + 1][0]);
                acc[mt + 1][1] = DT::mfma32(wf1, x1, acc[mt + 1][1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // epilogue: lane holds features m0 + 16 mt + 4 g .. + 3 of rows 16 rt + r16
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int64_t row = tile * ST_ROWS + rt * 16 + r16;
            const bool rv = row < a.rows;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int col = m0 + mt * 16 + 4 * g;
                const bool on = rv && col < a.M;
                const float4 bv = *reinterpret_cast<const float4*>(bl + mt * 16 + 4 * g);
                float o[4] = {acc[mt][rt][0] + bv.x, acc[mt][rt][1] + bv.y, acc[mt][rt][2] + bv.z, acc[mt][rt][3] + bv.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = keep_f32(apply_act16<ACT>(o[e]));
                if (AUX == 1 && on) {
                    const uint2 rv2 = *reinterpret_cast<const uint2*>(res + row * a.ldr + col);
                    o[0] += DT::to_f((u16)(rv2.x & 0xffff)); o[1] += DT::to_f((u16)(rv2.x >> 16));
                    o[2] += DT::to_f((u16)(rv2.y & 0xffff)); o[3] += DT::to_f((u16)(rv2.y >> 16));
                }
                if (AUX == 2 && on) {
                    const uint2 gv = *reinterpret_cast<const uint2*>(gate + row * a.ldgate + col);
                    if (!(DT::to_f((u16)(gv.x & 0xffff)) > 0.f)) o[0] = 0.f;
                    if (!(DT::to_f((u16)(gv.x >> 16)) > 0.f)) o[1] = 0.f;
                    if (!(DT::to_f((u16)(gv.y & 0xffff)) > 0.f)) o[2] = 0.f;
                    if (!(DT::to_f((u16)(gv.y >> 16)) > 0.f)) o[3] = 0.f;
                }
                uint2 ov;
                ov.x = DT::pack2(o[0], o[1]);
                ov.y = DT::pack2(o[2], o[3]);
                *reinterpret_cast<uint2*>(wt + r16 * TP + mt * 16 + 4 * g) = ov;
            }
            // the tile leaves row-major: 16-byte pieces, consecutive lanes on consecutive pieces of a row
            constexpr int OPR = MT * 2;                                   // 16-byte pieces per output row
#pragma unroll 1
            for (int c0 = 0; c0 < 16 * OPR; c0 += WAVE) {
                const int c = c0 + lane;
                const int r = c / OPR, pc = c % OPR;
                const int64_t orow = tile * ST_ROWS + rt * 16 + r;
                if (c < 16 * OPR && orow < a.rows && m0 + pc * 8 < a.M)
                    *reinterpret_cast<uint4*>(y + lin_yoff(a, orow) + m0 + pc * 8) = *reinterpret_cast<const uint4*>(wt + r * TP + pc * 8);
            }
        }
    }
}
#undef ST_FETCH

// ---- two Linears with a ReLU between them in one launch: y = (relu(x W1^T + b1)) W2^T + b2 ----------------------------
// The policy's token encoders (python/policy.py:1224-1249: Linear(in, d) ReLU Linear(d, d), in <= 64 lanes, padded to 64)
// as the streaming kernel twice over without the trip through HBM in between: both weights resident in LDS in fragment
// order, a wave streams 32-row tiles of x, and the first Linear's rounded output - the same 16 x d row tile that
// linear_stream_kernel would store - is read back from the wave's LDS tile as the second Linear's operand fragments.
// Every step is the arithmetic of the two separate launches (fp32 accumulate from zero in ascending k, + bias,
// ReLU, one rounding; fp32 accumulate, + bias, one rounding): the same bits.  Output rows may be grouped (LinArgs).
struct Mlp2Args {
    LinArgs l2;                  // the second Linear: w, bias, y / ldy / y_group / y_gstride, rows, K = M = d
    const void* x; int64_t ldx;  // (rows, 32 KC1) 16-bit
    const void* w1; const float* b1;      // (d, 32 KC1) 16-bit, (d) fp32
};

template <typename DT, int KC1, int KC, int MT>
__global__ __launch_bounds__(ST_THREADS) void mlp2_stream_kernel(Mlp2Args a, int walkers) {
    static_assert(MT * 16 == KC * 32, "the hidden width is the second Linear's K");
    extern __shared__ __attribute__((aligned(16))) uint4 wl[];   // W1 [MT * KC1][64], W2 [MT * KC][64], b1, b2, 8 wave tiles
    constexpr int KE = KC * 32, K1 = KC1 * 32;
    constexpr int TP = KE + 8;                                    // wave tile row pitch (elements)
    constexpr int PPR1 = K1 / 8;                                  // 16-byte pieces per x row
    constexpr int NLD = (16 * PPR1 + WAVE - 1) / WAVE;
    static_assert(16 * PPR1 == NLD * WAVE, "16 rows of x are whole wave loads");
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int walker = blockIdx.x;
    uint4* wl2 = wl + MT * KC1 * 64;
    {   // resident weights: fragment (mt, kc), lane l <- W[16 mt + l % 16][32 kc + 8 (l / 16) .. + 7]
        const u16* w1 = static_cast<const u16*>(a.w1);
        const u16* w2 = static_cast<const u16*>(a.l2.w);
        for (int i = tid; i < MT * KC1 * 64; i += ST_THREADS) {
            const int l = i & 63, f = i >> 6, mt = f / KC1, kc = f % KC1;
            wl[i] = *reinterpret_cast<const uint4*>(w1 + (int64_t)(mt * 16 + (l & 15)) * K1 + kc * 32 + 8 * (l >> 4));
        }
        for (int i = tid; i < MT * KC * 64; i += ST_THREADS) {
            const int l = i & 63, f = i >> 6, mt = f / KC, kc = f % KC;
            wl2[i] = *reinterpret_cast<const uint4*>(w2 + (int64_t)(mt * 16 + (l & 15)) * KE + kc * 32 + 8 * (l >> 4));
        }
    }
    float* bl1 = reinterpret_cast<float*>(wl2 + MT * KC * 64);
    float* bl2 = bl1 + MT * 16;
    u16* wt = reinterpret_cast<u16*>(bl2 + MT * 16) + wave * (16 * TP);
    for (int i = tid; i < MT * 16; i += ST_THREADS) { bl1[i] = a.b1[i]; bl2[i] = a.l2.bias[i]; }
    __syncthreads();                                              // the only barrier

    const u16* x = static_cast<const u16*>(a.x);
    u16* y = static_cast<u16*>(a.l2.y);
    const int64_t rows = a.l2.rows, ntiles = (rows + ST_ROWS - 1) / ST_ROWS;
    const int64_t stride = (int64_t)walkers * 8;
    int64_t tile = (int64_t)walker * 8 + wave;
    if (tile >= ntiles) return;
    u32x4 pa[NLD], pb[NLD];
#define M2_FETCH(t)                                                                                                   \
    _Pragma("unroll") for (int it = 0; it < NLD; ++it) {                                                               \
        const int p = it * WAVE + lane, r = p / PPR1, part = p % PPR1;                                                \
        int64_t ra = (t) * ST_ROWS + r, rb = ra + 16;                                                                 \
        ra = ra < rows ? ra : rows - 1;                                                                               \
        rb = rb < rows ? rb : rows - 1;                                                                               \
        pa[it] = *reinterpret_cast<const u32x4*>(x + ra * a.ldx + part * 8);                                          \
        pb[it] = *reinterpret_cast<const u32x4*>(x + rb * a.ldx + part * 8);                                          \
    }
    M2_FETCH(tile)
    for (; tile < ntiles; tile += stride) {
        u32x4 hf[2][KC];                                          // the hidden rows as operand fragments
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            // x rows -> fragments through the wave tile
            u32x4 xf[KC1];
#pragma unroll
            for (int it = 0; it < NLD; ++it) {
                const int p = it * WAVE + lane;
                *reinterpret_cast<u32x4*>(wt + (p / PPR1) * TP + (p % PPR1) * 8) = rt == 0 ? pa[it] : pb[it];
            }
#pragma unroll
            for (int kc = 0; kc < KC1; ++kc) xf[kc] = *reinterpret_cast<const u32x4*>(wt + r16 * TP + kc * 32 + 8 * g);
            // first Linear + ReLU, rounded, into the wave tile (row-major), two feature tiles at a time
#pragma unroll
            for (int mt = 0; mt < MT; mt += 2) {
                f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kc = 0; kc < KC1; ++kc) {
                    const s16x8 xv = __builtin_bit_cast(s16x8, xf[kc]);
                    a0 = DT::mfma32(__builtin_bit_cast(s16x8, wl[(mt * KC1 + kc) * 64 + lane]), xv, a0);
                    a1 = DT::mfma32(__builtin_bit_cast(s16x8, wl[((mt + 1) * KC1 + kc) * 64 + lane]), xv, a1);
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const f32x4 acc = h ? a1 : a0;
                    const float4 bv = *reinterpret_cast<const float4*>(bl1 + (mt + h) * 16 + 4 * g);
                    float o[4] = {acc[0] + bv.x, acc[1] + bv.y, acc[2] + bv.z, acc[3] + bv.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = keep_f32(apply_act16<BSRL_ACT_RELU>(o[e]));
                    uint2 ov;
                    ov.x = DT::pack2(o[0], o[1]);
                    ov.y = DT::pack2(o[2], o[3]);
                    *reinterpret_cast<uint2*>(wt + r16 * TP + (mt + h) * 16 + 4 * g) = ov;
                }
            }
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) hf[rt][kc] = *reinterpret_cast<const u32x4*>(wt + r16 * TP + kc * 32 + 8 * g);
        }
        M2_FETCH(tile + stride)                                   // rows past the end clamp to the last row
        // second Linear
        f32x4 acc[MT][2];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) { acc[mt][0] = (f32x4){0.f, 0.f, 0.f, 0.f}; acc[mt][1] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) {
            const s16x8 x0 = __builtin_bit_cast(s16x8, hf[0][kc]), x1 = __builtin_bit_cast(s16x8, hf[1][kc]);
#pragma unroll
            for (int mt = 0; mt < MT; mt += 2) {
                const s16x8 wf0 = __builtin_bit_cast(s16x8, wl2[(mt * KC + kc) * 64 + lane]);
                const s16x8 wf1 = __builtin_bit_cast(s16x8, wl2[((mt + 1) * KC + kc) * 64 + lane]);
                acc[mt][0] = DT::mfma32(wf0, x0, acc[mt][0]);
                acc[mt][1] = DT::mfma32(wf0, x1, acc[mt][1]);
                acc[mt + 1][0] = DT::mfma32(wf1, x0, acc[mt + 1][0]);
                acc[mt + 1][1] = DT::mfma32(wf1, x1, acc[mt + 1][1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const float4 bv = *reinterpret_cast<const float4*>(bl2 + mt * 16 + 4 * g);
                float o[4] = {acc[mt][rt][0] + bv.x, acc[mt][rt][1] + bv.y, acc[mt][rt][2] + bv.z, acc[mt][rt][3] + bv.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = keep_f32(o[e]);
                uint2 ov;
                ov.x = DT::pack2(o[0], o[1]);
                ov.y = DT::pack2(o[2], o[3]);
                *reinterpret_cast<uint2*>(wt + r16 * TP + mt * 16 + 4 * g) = ov;
            }
            constexpr int OPR = MT * 2;                           // 16-byte pieces per output row
#pragma unroll 1
            for (int c0 = 0; c0 < 16 * OPR; c0 += WAVE) {
                const int c = c0 + lane;
                const int r = c / OPR, pc = c % OPR;
                const int64_t orow = tile * ST_ROWS + rt * 16 + r;
                if (c < 16 * OPR && orow < rows)
                    *reinterpret_cast<uint4*>(y + lin_yoff(a.l2, orow) + pc * 8) = *reinterpret_cast<const uint4*>(wt + r * TP + pc * 8);
            }
        }
    }
}
#undef M2_FETCH

int device_cus() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        return n;
    }();
    return cus;
}

template <typename DT, int KC, int MT, int ACT, int AUX>
bool launch(const LinArgs& a, hipStream_t st) {
    constexpr int TP = (KC * 32 > MT * 16 ? KC * 32 : MT * 16) + 8;
    const size_t lds = (size_t)MT * KC * 1024 + (size_t)MT * 16 * sizeof(float) + (size_t)8 * 16 * TP * sizeof(u16);
    auto kern = linear_stream_kernel<DT, KC, MT, ACT, AUX>;
    // workgroups resident per CU (LDS and registers), 0 = this instantiation cannot run here
    static const int per_cu = [&] {
        int n = 0;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, ST_THREADS, lds) != hipSuccess) return 0;
        return n;
    }();
    if (per_cu < 1) return false;
    const int nb = (a.M + MT * 16 - 1) / (MT * 16);
    const int64_t ntiles = (a.rows + ST_ROWS - 1) / ST_ROWS;
    // every workgroup must be resident at once (the rows are split statically); the walkers of a column block come
    // in whole groups of 8 block ids (one per XCD)
    const int64_t slots = (int64_t)device_cus() * per_cu;
    int64_t walkers = slots / nb / 8 * 8;
    if (walkers < 8) return false;
    const int64_t need = ((ntiles + 7) / 8 + 7) / 8 * 8;
    if (walkers > need) walkers = need;
    hipLaunchKernelGGL(kern, dim3((unsigned)(walkers * nb)), dim3(ST_THREADS), lds, st, a, nb, (int)walkers);
    return true;
}

template <typename DT, int ACT, int AUX>
bool by_k(const LinArgs& a, hipStream_t st) {
    switch (a.K / 32) {
        case 4: return launch<DT, 4, 8, ACT, AUX>(a, st);
        case 6: return launch<DT, 6, 12, ACT, AUX>(a, st);
        case 8: return launch<DT, 8, 8, ACT, AUX>(a, st);
        default: return false;
    }
}

template <typename DT>
bool dispatch(const LinArgs& a, int act, hipStream_t st) {
    // the combinations the policy uses: any activation alone, a residual without one, the gate without one
    if (a.res && a.gate) return false;
    if (a.gate) return act == BSRL_ACT_NONE ? by_k<DT, BSRL_ACT_NONE, 2>(a, st) : false;
    if (a.res) return act == BSRL_ACT_NONE ? by_k<DT, BSRL_ACT_NONE, 1>(a, st) : false;
    if (act == BSRL_ACT_RELU) return by_k<DT, BSRL_ACT_RELU, 0>(a, st);
    if (act == BSRL_ACT_GELU) return by_k<DT, BSRL_ACT_GELU, 0>(a, st);
    return by_k<DT, BSRL_ACT_NONE, 0>(a, st);
}


template <typename DT, int KC, int MT>
bool mlp2_launch(const Mlp2Args& a, hipStream_t st) {
    constexpr int KC1 = 2, TP = KC * 32 + 8;
    const size_t lds = (size_t)MT * (KC1 + KC) * 1024 + (size_t)2 * MT * 16 * sizeof(float) + (size_t)8 * 16 * TP * sizeof(u16);
    auto kern = mlp2_stream_kernel<DT, KC1, KC, MT>;
    static const bool ready = [&] {
        return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess;
    }();
    if (!ready) { (void)hipGetLastError(); return false; }
    const int64_t ntiles = (a.l2.rows + ST_ROWS - 1) / ST_ROWS;
    int64_t walkers = device_cus();                               // one workgroup per CU (the resident weights fill its LDS)
    const int64_t need = (ntiles + 7) / 8;
    if (walkers > need) walkers = need;
    hipLaunchKernelGGL(kern, dim3((unsigned)walkers), dim3(ST_THREADS), lds, st, a, (int)walkers);
    return true;
}
}  // namespace

bool bsrl_linear_stream(const LinArgs& a, int act, int dtype, hipStream_t st) {
    // many rows, K = 128 / 192 / 256, 16-bit in and out, 16-byte aligned rows
    if (a.out_f32 || a.y2 || a.rows < 8192 || a.K % 32 != 0 || a.M % 8 != 0) return false;
    if (a.ldx % 8 != 0 || !bsrl_aligned(a.x, 16) || !bsrl_aligned(a.w, 16)) return false;
    if (a.ldy % 8 != 0 || a.y_gstride % 8 != 0 || !bsrl_aligned(a.y, 16)) return false;
    if (a.res && (a.ldr % 4 != 0 || !bsrl_aligned(a.res, 8))) return false;
    if (a.gate && (a.ldgate % 4 != 0 || !bsrl_aligned(a.gate, 8))) return false;
    if (a.bias && !bsrl_aligned(a.bias, 4)) return false;
    return dtype == BSRL_F16 ? dispatch<F16>(a, act, st) : dispatch<BF16>(a, act, st);
}

bool bsrl_mlp2_stream(const LinArgs& l2, const void* x, int64_t ldx, const void* w1, const float* b1, int64_t K1, int dtype,
                      hipStream_t st) {
    // 64 input lanes, d = 128 / 192, 16-bit in and out, 16-byte aligned rows, both biases present
    if (K1 != 64 || l2.K != l2.M || (l2.M != 128 && l2.M != 192) || l2.out_f32 || l2.y2 || l2.res || l2.gate || !l2.bias || !b1) return false;
    if (ldx % 8 != 0 || !bsrl_aligned(x, 16) || !bsrl_aligned(w1, 16) || !bsrl_aligned(l2.w, 16)) return false;
    if (l2.ldy % 8 != 0 || l2.y_gstride % 8 != 0 || !bsrl_aligned(l2.y, 16) || l2.rows < 1 || l2.rows > 0x7fffffffLL) return false;
    Mlp2Args a{l2, x, ldx, w1, b1};
    if (dtype == BSRL_F16) return l2.M == 128 ? mlp2_launch<F16, 4, 8>(a, st) : mlp2_launch<F16, 6, 12>(a, st);
    return l2.M == 128 ? mlp2_launch<BF16, 4, 8>(a, st) : mlp2_launch<BF16, 6, 12>(a, st);
}
