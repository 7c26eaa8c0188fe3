// Weight / bias gradient of a Linear on the 16-bit stream: dW = dy^T x, db = column sums of dy.
//
// Replaces fp16_gemm.wgrad / wgrad_bgrad (reference python/beat_arena_env/csrc/fp16_gemm.cu:189-277,
// 404-476; callers python/fp16_linear.py:442-458): dy (rows, M), x (rows, K) in fp16 / bf16, fp32
// accumulation, fp32 outputs dW (M, K) and db (M).
//
// The contraction runs over ROWS, so both MFMA operands are needed "k-contiguous per lane" while
// memory holds them row-major.  Tiles of 32 rows are copied to LDS as they lie (16-byte coalesced
// loads, 16-byte LDS writes) and the fragments come out through the LDS transpose load
// (ds_read_b64_tr_b16): within a group of 16 lanes, lanes 4j..4j+3 present row j (4 x 4 elements)
// and lane i receives element i of rows 0..3 - four consecutive contraction indices of one column,
// i.e. half of a v_mfma_f32_16x16x32 fragment per instruction, no 16-bit gathers.
//
// Workgroup = 4 waves, output tile 128 (M) x 128 (K), wave tile 64 x 64 (4 x 4 accumulators); each
// 32-row step costs a wave 8 transpose loads per operand for 16 MFMAs.  db is one more MFMA per
// A fragment against an all-ones B fragment (the tile column 0 workgroups only): the bias gradient
// rides the matrix pipe instead of a separate column-sum pass over dy.
// The output is small (M x K <= a few 100k) and the rows are many: the grid splits the rows into
// S chunks per tile; split s of every tile is mapped to consecutive block ids of ONE XCD (id % 8),
// so the tiles that re-read the same dy / x rows share that XCD's L2.  Partials land in the
// caller's workspace and a second kernel folds them in a fixed order (reproducible, no atomics).
// One step of both operands is prefetched in registers; a 3-step register ring was measured and dropped: at 206
// VGPRs two workgroups fit a CU instead of four and the kernel ran 1.5 - 1.8x slower - occupancy, not prefetch
// depth, is what hides the step latency here.
#include "bsrl_common.h"

namespace {

constexpr int STEP = 32;                                // rows per LDS step
constexpr int MAX_SPLIT = 512;
// Output tile edge per dimension: 128 or 192, whichever pads the dimension less (192 on a tie: fewer tiles).  A
// workgroup re-reads its dy and x column slabs once per tile of the other dimension, and what bounds this kernel
// is the rate at which the CUs pull those slabs from L2 (~7.5 TB/s chip-wide measured: 576 x 192 as 5 x 2 tiles of
// 128 moved 5 KB per row for 1.5 KB of operands); 192-wide tiles cover the d = 192 shapes in 3 x 1 / 4 x 1 / 1 x 1
// tiles with no padding.
inline int tile_edge(int64_t dim) {
    const int64_t p192 = (dim + 191) / 192 * 192, p128 = (dim + 127) / 128 * 128;
    return p192 <= p128 ? 192 : 128;
}

struct WgArgs {
    const u16* dy; int64_t lddy; const u16* x; int64_t ldx;
    float* dw; float* db; float* part;                  // part: [S][M*K (+ M)] when S > 1
    int64_t rows; int M, K, S, tiles_m, tiles_n; int64_t rows_per_split;
    int vec_ok;                                         // every 8-element piece may be one 16-byte load
};

typedef short s16x4v __attribute__((ext_vector_type(4)));

template <int PITCH>
__device__ __forceinline__ s16x8 tr_frag(const u16* tile, int row0, int col0, int lane) {
    // lane (i = lane % 16, g = lane / 16): rows row0 + 8 g + {0..3 | 4..7}, presents 4 elements at column col0 + 4 (i % 4) of row (i / 4)
    const int i = lane & 15, g = lane >> 4;
    const u16* p = tile + (row0 + 8 * g + (i >> 2)) * PITCH + col0 + 4 * (i & 3);
    typedef __attribute__((address_space(3))) s16x4v* lptr;
    const s16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p));
    const s16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p + 4 * PITCH));
    return (s16x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

template <typename DT, int WG_M, int WG_N>
__global__ __launch_bounds__(256, (WG_M * WG_N > 128 * 128 ? 2 : 1)) void wgrad_kernel(WgArgs a) {
    // LDS row pitches (elements): rows 32 B (128-wide) or 160 B (192-wide) apart modulo 256 B - either way 8
    // consecutive rows start on 8 different 32-byte bank groups
    constexpr bool BIG = WG_M == 192 || WG_N == 192;
    constexpr int PY = WG_M + 16, PX = WG_N + 16;
    constexpr int TILE_Y = STEP * PY, TILE_X = STEP * PX;
    constexpr int MI = WG_M / 32, NI = WG_N / 32;                // accumulator tiles per wave: MI x NI
    constexpr int LJY = STEP * (WG_M / 8) / 256, LJX = STEP * (WG_N / 8) / 256;    // 16-byte pieces per thread and step
    __shared__ __attribute__((aligned(16))) u16 lds[2 * (TILE_Y + TILE_X)];        // [buffer][dy | x]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    // block id -> (split, tile): ids with equal id % 8 (one XCD) walk the tiles of one split back to back
    const int T = a.tiles_m * a.tiles_n;
    const int b = blockIdx.x;
    const int xcd = b & 7, q = b >> 3;
    const int tile = q % T, split = (q / T) * 8 + xcd;
    if (split >= a.S) return;
    const int tm = tile / a.tiles_n, tn = tile % a.tiles_n;
    const int m0 = tm * WG_M, n0 = tn * WG_N;
    const int64_t r_begin = (int64_t)split * a.rows_per_split;
    const int64_t r_end = r_begin + a.rows_per_split < a.rows ? r_begin + a.rows_per_split : a.rows;
    const bool want_db = a.db != nullptr && tn == 0 && wn == 0;

    // loader: piece p = tid + 256 j of a tile is (row p / (W / 8), columns 8 (p % (W / 8)) .. + 7)
    uint4 ry[LJY], rx[LJX];
    auto piece = [&](const u16* base, int64_t ld, int64_t row, int col, int ncols) -> uint4 {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (row < r_end && col < ncols) {
            const u16* p = base + row * ld + col;
            if (BIG || a.vec_ok) v = *reinterpret_cast<const uint4*>(p);      // 192-wide tiles are only launched on 16-byte-aligned operands
            else {
                u16 e[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) e[k] = col + k < ncols ? p[k] : (u16)0;
                v = make_uint4(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16),
                               e[4] | ((uint32_t)e[5] << 16), e[6] | ((uint32_t)e[7] << 16));
            }
        }
        return v;
    };
    auto gload = [&](int64_t r0) {
#pragma unroll
        for (int j = 0; j < LJY; ++j) {
            const int p = tid + 256 * j;
            ry[j] = piece(a.dy, a.lddy, r0 + p / (WG_M / 8), m0 + 8 * (p % (WG_M / 8)), a.M);
        }
#pragma unroll
        for (int j = 0; j < LJX; ++j) {
            const int p = tid + 256 * j;
            rx[j] = piece(a.x, a.ldx, r0 + p / (WG_N / 8), n0 + 8 * (p % (WG_N / 8)), a.K);
        }
    };
    auto lstore = [&](int buf) {
        u16* ty = lds + buf * (TILE_Y + TILE_X);
        u16* tx = ty + TILE_Y;
#pragma unroll
        for (int j = 0; j < LJY; ++j) {
            const int p = tid + 256 * j;
            *reinterpret_cast<uint4*>(ty + (p / (WG_M / 8)) * PY + 8 * (p % (WG_M / 8))) = ry[j];
        }
#pragma unroll
        for (int j = 0; j < LJX; ++j) {
            const int p = tid + 256 * j;
            *reinterpret_cast<uint4*>(tx + (p / (WG_N / 8)) * PX + 8 * (p % (WG_N / 8))) = rx[j];
        }
    };

    f32x4 acc[MI][NI], accb[MI];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        accb[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    const u16 one = DT::from_f(1.0f);
    const s16x8 ones = {(short)one, (short)one, (short)one, (short)one, (short)one, (short)one, (short)one, (short)one};

    const int nsteps = (int)((r_end - r_begin + STEP - 1) / STEP);
    if (nsteps > 0) gload(r_begin);
    for (int s = 0; s < nsteps; ++s) {
        const int buf = s & 1;
        lstore(buf);
        __syncthreads();                               // step s visible; everyone is past step s - 1's reads of the other buffer
        if (s + 1 < nsteps) gload(r_begin + (int64_t)(s + 1) * STEP);
        const u16* ty = lds + buf * (TILE_Y + TILE_X);
        const u16* tx = ty + TILE_Y;
#pragma unroll
        for (int c = 0; c < STEP / 32; ++c) {
            // the x fragments stay for the whole chunk; the dy fragments pass through two at a time
            s16x8 fb[NI];
#pragma unroll
            for (int j = 0; j < NI; ++j) fb[j] = tr_frag<PX>(tx, 32 * c, wn * (WG_N / 2) + 16 * j, lane);
#pragma unroll
            for (int i0 = 0; i0 < MI; i0 += 2) {
                s16x8 fa[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) fa[u] = tr_frag<PY>(ty, 32 * c, wm * (WG_M / 2) + 16 * (i0 + u), lane);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
#pragma unroll
                    for (int j = 0; j < NI; ++j) acc[i0 + u][j] = DT::mfma32(fa[u], fb[j], acc[i0 + u][j]);
                    if (want_db) accb[i0 + u] = DT::mfma32(fa[u], ones, accb[i0 + u]);
                }
                if (MI > 4) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // lane holds D[m = 4 (lane / 16) + e][n = lane % 16] of each 16 x 16 tile
    float* out = a.S > 1 ? a.part + (int64_t)split * ((int64_t)a.M * a.K + a.M) : a.dw;
    float* outb = a.S > 1 ? out + (int64_t)a.M * a.K : a.db;
    const int i16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wm * (WG_M / 2) + 16 * i + 4 * g + e;
            if (m >= a.M) continue;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int n = n0 + wn * (WG_N / 2) + 16 * j + i16;
                if (n < a.K) out[(int64_t)m * a.K + n] = acc[i][j][e];
            }
            if (want_db && i16 == 0) outb[m] = accb[i][e];
        }
    }
}

// dW / db = sum over splits of the partials.  A block owns 32 consecutive outputs (one 128-byte line per split);
// thread (e, sg) = (tid % 32, tid / 32) adds the splits sg, sg + 8, ... in that order and the 8 group sums are
// added in group order: a fixed order for a given split count, no atomics.  (One thread per output walking all
// splits took 120 us at 512 splits of a 192 x 192 output - 75 MB - for a 45 us main kernel.)
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ part, int S, int64_t n_w, int M,
                                                           float* __restrict__ dw, float* __restrict__ db) {
    __shared__ float sums[8][33];
    const int e = threadIdx.x & 31, sg = threadIdx.x >> 5;
    const int64_t i = (int64_t)blockIdx.x * 32 + e;
    const int64_t n = n_w + (db ? M : 0), stride = n_w + M;
    float t = 0.f;
    if (i < n) {
        const float* p = part + i;
        int sp = sg;
        for (; sp + 24 < S; sp += 32) {
            const float v0 = p[(int64_t)sp * stride], v1 = p[(int64_t)(sp + 8) * stride];
            const float v2 = p[(int64_t)(sp + 16) * stride], v3 = p[(int64_t)(sp + 24) * stride];
            t += v0; t += v1; t += v2; t += v3;
        }
        for (; sp < S; sp += 8) t += p[(int64_t)sp * stride];
    }
    sums[sg][e] = t;
    __syncthreads();
    if (sg == 0 && i < n) {
        float r = sums[0][e];
#pragma unroll
        for (int k = 1; k < 8; ++k) r += sums[k][e];
        if (i < n_w) dw[i] = r; else db[i - n_w] = r;
    }
}

// upper bound of the split count for an output of `tiles` tiles, `big` when any tile edge is 192 (two workgroups
// fit a CU then, four otherwise)
int split_cap(int tiles, bool big) {
    // splits x tiles fills the chip's workgroup slots once and never spills into a second, nearly empty round:
    // rounded DOWN to the multiple of 8 the XCD mapping launches anyway
    int64_t s = (big ? 512 : 1024) / tiles;
    if (s > 8) s = s / 8 * 8;
    if (s > MAX_SPLIT) s = MAX_SPLIT;
    return s < 1 ? 1 : (int)s;
}

int plan_splits(int64_t rows, int tiles, bool big) {
    int64_t s = split_cap(tiles, big);
    const int64_t by_rows = (rows + 4 * STEP - 1) / (4 * STEP);      // at least 4 steps per split
    if (s > by_rows) s = by_rows;
    return s < 1 ? 1 : (int)s;
}

}  // namespace

extern "C" int64_t bsrl_wgrad_workspace_size(int64_t M, int64_t K) {
    if (M <= 0 || K <= 0) return 0;
    const int em = tile_edge(M), en = tile_edge(K);
    const int64_t T = ((M + em - 1) / em) * ((K + en - 1) / en);
    if (T > (1 << 20)) return 0;
    return (int64_t)split_cap((int)T, em == 192 || en == 192) * (M * K + M) * (int64_t)sizeof(float);
}

extern "C" int bsrl_wgrad(const void* dy, int64_t lddy, const void* x, int64_t ldx, float* dw, float* db,
                          void* workspace, int64_t rows, int64_t M, int64_t K, int dtype, bsrl_stream stream) {
    if (!dw || !workspace || (rows > 0 && (!dy || !x))) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: null pointer");
    if (rows < 0 || M < 1 || K < 1 || M > 65536 || K > 65536 || lddy < M || ldx < K)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: need rows >= 0, 1 <= M, K <= 65536 and row pitches >= the widths");
    if (dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: dtype must be F16 or BF16 (got %d)", dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool vec_ok = M % 8 == 0 && K % 8 == 0 && lddy % 8 == 0 && ldx % 8 == 0 && bsrl_aligned(dy, 16) && bsrl_aligned(x, 16);
    // 128-wide tiles on unaligned operands use fewer splits than the workspace bound, never more
    const int em = vec_ok ? tile_edge(M) : 128, en = vec_ok ? tile_edge(K) : 128;
    const bool big = em == 192 || en == 192;
    const int tiles_m = (int)((M + em - 1) / em), tiles_n = (int)((K + en - 1) / en);
    const int T = tiles_m * tiles_n;
    if (T > (1 << 20)) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: M x K too large");
    WgArgs a;
    a.dy = static_cast<const u16*>(dy); a.lddy = lddy; a.x = static_cast<const u16*>(x); a.ldx = ldx;
    a.dw = dw; a.db = db; a.part = static_cast<float*>(workspace);
    a.rows = rows; a.M = (int)M; a.K = (int)K; a.tiles_m = tiles_m; a.tiles_n = tiles_n;
    a.S = plan_splits(rows, T, big);
    const int64_t ws_splits = bsrl_wgrad_workspace_size(M, K) / ((M * K + M) * (int64_t)sizeof(float));
    if (a.S > ws_splits) a.S = (int)ws_splits;         // the caller's workspace was sized by that function
    const int64_t steps = (rows + STEP - 1) / STEP;
    a.rows_per_split = ((steps + a.S - 1) / a.S) * STEP;
    a.vec_ok = vec_ok;
    // S rounded up to whole groups of 8 so that every XCD walks complete splits; surplus blocks exit at once
    const int64_t grid = (int64_t)((a.S + 7) / 8) * 8 * T;
    if (grid > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: grid too large");
#define WG_GO(DT, TM_, TN_) hipLaunchKernelGGL((wgrad_kernel<DT, TM_, TN_>), dim3((unsigned)grid), dim3(256), 0, st, a)
#define WG_PICK(DT) do { if (em == 192) { if (en == 192) WG_GO(DT, 192, 192); else WG_GO(DT, 192, 128); } \
                         else { if (en == 192) WG_GO(DT, 128, 192); else WG_GO(DT, 128, 128); } } while (0)
    if (dtype == BSRL_F16) WG_PICK(F16); else WG_PICK(BF16);
#undef WG_PICK
#undef WG_GO
    if (a.S > 1) {
        const int64_t n = M * K + (db ? M : 0);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((n + 31) / 32)), dim3(256), 0, st,
                           a.part, a.S, M * K, (int)M, dw, db);
    }
    BSRL_CHECK_LAUNCH("bsrl_wgrad");
    return BSRL_OK;
}
