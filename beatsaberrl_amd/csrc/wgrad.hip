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
// caller's workspace and a second kernel folds them in split order (reproducible, no atomics).
// One step of both operands is prefetched in registers; a 3-step register ring was measured and dropped: at 206
// VGPRs two workgroups fit a CU instead of four and the kernel ran 1.5 - 1.8x slower - occupancy, not prefetch
// depth, is what hides the step latency here.
#include "bsrl_common.h"

namespace {

constexpr int WG_M = 128, WG_N = 128, STEP = 32;      // output tile and rows per LDS step
constexpr int PITCH = WG_M + 16;                        // LDS row pitch (elements): rows 32 B apart modulo 256 B
constexpr int LJ = STEP / 16;                           // 16-byte pieces per thread and tile
constexpr int TILE_E = STEP * PITCH;                    // one operand tile (elements)
constexpr int MAX_SPLIT = 128;

struct WgArgs {
    const u16* dy; int64_t lddy; const u16* x; int64_t ldx;
    float* dw; float* db; float* part;                  // part: [S][M*K (+ M)] when S > 1
    int64_t rows; int M, K, S, tiles_m, tiles_n; int64_t rows_per_split;
    int vec_ok;                                         // every 8-element piece may be one 16-byte load
};

typedef short s16x4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ s16x8 tr_frag(const u16* tile, int row0, int col0, int lane) {
    // lane (i = lane % 16, g = lane / 16): rows row0 + 8 g + {0..3 | 4..7}, presents 4 elements at column col0 + 4 (i % 4) of row (i / 4)
    const int i = lane & 15, g = lane >> 4;
    const u16* p = tile + (row0 + 8 * g + (i >> 2)) * PITCH + col0 + 4 * (i & 3);
    typedef __attribute__((address_space(3))) s16x4v* lptr;
    const s16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p));
    const s16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(p + 4 * PITCH));
    return (s16x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

template <typename DT>
__global__ __launch_bounds__(256) void wgrad_kernel(WgArgs a) {
    __shared__ __attribute__((aligned(16))) u16 lds[2 * 2 * TILE_E];   // [buffer][dy | x]
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

    // loader: a thread owns pieces (row = tid / 16 + 16 j, columns 8 (tid % 16) .. + 7), j < LJ, of both tiles
    const int lr = tid >> 4, lc = 8 * (tid & 15);
    uint4 ry[LJ], rx[LJ];
    auto piece = [&](const u16* base, int64_t ld, int64_t row, int col, int ncols) -> uint4 {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (row < r_end && col < ncols) {
            const u16* p = base + row * ld + col;
            if (a.vec_ok) v = *reinterpret_cast<const uint4*>(p);
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
        for (int j = 0; j < LJ; ++j) {
            ry[j] = piece(a.dy, a.lddy, r0 + lr + 16 * j, m0 + lc, a.M);
            rx[j] = piece(a.x, a.ldx, r0 + lr + 16 * j, n0 + lc, a.K);
        }
    };
    auto lstore = [&](int buf) {
        u16* ty = lds + buf * 2 * TILE_E;
        u16* tx = ty + TILE_E;
#pragma unroll
        for (int j = 0; j < LJ; ++j) {
            *reinterpret_cast<uint4*>(ty + (lr + 16 * j) * PITCH + lc) = ry[j];
            *reinterpret_cast<uint4*>(tx + (lr + 16 * j) * PITCH + lc) = rx[j];
        }
    };

    f32x4 acc[4][4], accb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        accb[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
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
        const u16* ty = lds + buf * 2 * TILE_E;
        const u16* tx = ty + TILE_E;
#pragma unroll
        for (int c = 0; c < STEP / 32; ++c) {
            s16x8 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = tr_frag(ty, 32 * c, wm * 64 + 16 * i, lane);
#pragma unroll
            for (int j = 0; j < 4; ++j) fb[j] = tr_frag(tx, 32 * c, wn * 64 + 16 * j, lane);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = DT::mfma32(fa[i], fb[j], acc[i][j]);
            if (want_db) {
#pragma unroll
                for (int i = 0; i < 4; ++i) accb[i] = DT::mfma32(fa[i], ones, accb[i]);
            }
        }
    }

    // lane holds D[m = 4 (lane / 16) + e][n = lane % 16] of each 16 x 16 tile
    float* out = a.S > 1 ? a.part + (int64_t)split * ((int64_t)a.M * a.K + a.M) : a.dw;
    float* outb = a.S > 1 ? out + (int64_t)a.M * a.K : a.db;
    const int i16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wm * 64 + 16 * i + 4 * g + e;
            if (m >= a.M) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn * 64 + 16 * j + i16;
                if (n < a.K) out[(int64_t)m * a.K + n] = acc[i][j][e];
            }
            if (want_db && i16 == 0) outb[m] = accb[i][e];
        }
    }
}

// dW / db = sum over splits of the partials, in split order
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ part, int S, int64_t n_w, int M,
                                                           float* __restrict__ dw, float* __restrict__ db) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n = n_w + (db ? M : 0), stride = n_w + M;
    if (i >= n) return;
    float t = 0.f;
    for (int s = 0; s < S; ++s) t += part[(int64_t)s * stride + i];
    if (i < n_w) dw[i] = t; else db[i - n_w] = t;
}

int plan_splits(int64_t rows, int tiles) {
    int64_t s = (1024 + tiles - 1) / tiles;                         // ~4 workgroups per CU in flight
    const int64_t by_rows = (rows + 4 * STEP - 1) / (4 * STEP);      // at least 4 steps per split
    if (s > by_rows) s = by_rows;
    if (s > MAX_SPLIT) s = MAX_SPLIT;
    return s < 1 ? 1 : (int)s;
}

}  // namespace

extern "C" int64_t bsrl_wgrad_workspace_size(int64_t M, int64_t K) {
    if (M <= 0 || K <= 0) return 0;
    return (int64_t)MAX_SPLIT * (M * K + M) * (int64_t)sizeof(float);
}

extern "C" int bsrl_wgrad(const void* dy, int64_t lddy, const void* x, int64_t ldx, float* dw, float* db,
                          void* workspace, int64_t rows, int64_t M, int64_t K, int dtype, bsrl_stream stream) {
    if (!dw || !workspace || (rows > 0 && (!dy || !x))) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: null pointer");
    if (rows < 0 || M < 1 || K < 1 || M > 65536 || K > 65536 || lddy < M || ldx < K)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: need rows >= 0, 1 <= M, K <= 65536 and row pitches >= the widths");
    if (dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: dtype must be F16 or BF16 (got %d)", dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int tiles_m = (int)((M + WG_M - 1) / WG_M), tiles_n = (int)((K + WG_N - 1) / WG_N);
    const int T = tiles_m * tiles_n;
    if (T > (1 << 20)) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: M x K too large");
    WgArgs a;
    a.dy = static_cast<const u16*>(dy); a.lddy = lddy; a.x = static_cast<const u16*>(x); a.ldx = ldx;
    a.dw = dw; a.db = db; a.part = static_cast<float*>(workspace);
    a.rows = rows; a.M = (int)M; a.K = (int)K; a.tiles_m = tiles_m; a.tiles_n = tiles_n;
    a.S = plan_splits(rows, T);
    const int64_t steps = (rows + STEP - 1) / STEP;
    a.rows_per_split = ((steps + a.S - 1) / a.S) * STEP;
    a.vec_ok = M % 8 == 0 && K % 8 == 0 && lddy % 8 == 0 && ldx % 8 == 0 && bsrl_aligned(dy, 16) && bsrl_aligned(x, 16);
    // S rounded up to whole groups of 8 so that every XCD walks complete splits; surplus blocks exit at once
    const int64_t grid = (int64_t)((a.S + 7) / 8) * 8 * T;
    if (grid > 0x7fffffff) BSRL_FAIL(BSRL_EINVAL, "bsrl_wgrad: grid too large");
    if (dtype == BSRL_F16) hipLaunchKernelGGL(wgrad_kernel<F16>, dim3((unsigned)grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(wgrad_kernel<BF16>, dim3((unsigned)grid), dim3(256), 0, st, a);
    if (a.S > 1) {
        const int64_t n = M * K + (db ? M : 0);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                           a.part, a.S, M * K, (int)M, dw, db);
    }
    BSRL_CHECK_LAUNCH("bsrl_wgrad");
    return BSRL_OK;
}
