// Ring-buffered MFMA linear for large row counts: y = act(x W^T + b) (+ residual) (* gate), 16-bit in / out.
//
// The operands never pass through registers: every 1 KB operand block is fetched by ONE wave instruction that
// writes straight into LDS (global_load_lds_dwordx4: lane l's 16 bytes land at slot l of the block), into a ring of
// NS stages of BK k each; loads run NS - 1 stages ahead of the MFMAs and there is one barrier per stage.  No load
// needs a VALU op in the loop: the per-lane offsets are fixed and the k advance happens on the scalar base address.
// A wave owns 64 rows x 128 columns (4 x 8 accumulator tiles, 32 MFMAs per 32 k against 12 fragment reads).
//
// Block layouts (conflict-free for the 8 lanes a ds_read_b128 serves per cycle, and contiguous in memory per row):
//   BK = 32: a block is 16 rows x 64 B; lane l fetches row l / 4, k piece (l % 4) ^ ((row / 2) % 4);
//   BK = 64: a block is 8 rows x 128 B (whole cache lines: half as many requests to L2, ~11 % faster per k);
//            lane l fetches row l / 8, k piece (l % 8) ^ row.
//
// Three geometries, picked by the column count:
//   narrow: 256 x 128 tile, 4 waves, BK 32 x 3 stages = 72 KB, two workgroups per CU (the epilogue and ring fill
//           of one overlap the main loop of the other);
//   wide:   256 x 256 tile, 8 waves (4 row slabs x 2 column slabs), BK 64 x 2 stages = 128 KB, one workgroup per
//           CU.  What bounds the main loop is the rate at which a CU pulls operands from L2 (~16 B/clk/CU measured
//           with either geometry, against 48 B/clk that 256 x 128 tiles would need at full MFMA rate and 32 for
//           256 x 256): a stage of the wide tile moves 2/3 of the bytes per MFMA.
//   192:    256 x 192 tile, 8 waves of 64 x 96, BK 64 x 2 stages = 112 KB: one column block for the d = 192
//           shapes, where 128-column tiles take two (the second half empty) and pull x from L2 twice.
// Workgroup ids are remapped so that all column blocks of a row block run on the same XCD one after the other:
// the row block's x tile crosses the fabric once and then hits in that XCD's L2.
//
// Epilogue: accumulators are transposed through LDS (fp32) so that 16 lanes own one 256-byte row segment: 16-byte
// residual / gate loads and stores of whole segments.  All 16 residual (or gate) loads of a wave tile are issued
// before the first of them is needed; issued one row group at a time, each paid its full memory latency and the
// epilogue took as long as 20 k-stages.
//
// Same arithmetic contract as the other 16-bit linear kernels (fp32 accumulate in fixed k order, a row's result
// independent of the batch): interchangeable with them, the entry point picks by shape.
#include "linear_args.h"

namespace {

constexpr int BM = 256;
constexpr int EP_LD = 128 + 4;                                // epilogue row pitch (floats): a wave stages 16 x <= 128

// Geometry of one instantiation: WC wave columns of 16 CT (workgroup tile 256 x 16 CT WC, 4 WC waves), BK k per
// stage (32: a load covers 16 rows x 64 B; 64: 8 rows x 128 B), NS stages.
template <int WC, int BK, int NS, int CT = 8>
struct Geo {
    static constexpr int CW = 16 * CT;                                   // columns per wave
    static constexpr int BN = CW * WC, NW = 4 * WC, NT = 64 * NW;
    static constexpr int KCH = BK / 32;                                  // 32-wide k chunks per stage
    static constexpr int RPL = 512 / BK, LPR = 64 / RPL;                 // rows per load instruction, lanes per row
    static constexpr int XB = BM / RPL, WB = BN / RPL, NB = XB + WB;     // 1 KB blocks per stage
    static constexpr int STAGE_U4 = NB * 64;
    static constexpr int LDS_BYTES = NS * STAGE_U4 * 16;
    static constexpr int NLX = XB / NW, NLW = WB / NW, NLD = NLX + NLW;  // loads per wave and stage
    static constexpr int WG_PER_CU = LDS_BYTES <= 80 * 1024 ? 2 : 1;
    static_assert(XB % NW == 0 && WB % NW == 0, "blocks must divide over the waves");
    static_assert(NLD <= KCH * CT, "a stage's loads are spread over its MFMA groups");
    static_assert(16 * EP_LD * 4 * NW <= LDS_BYTES, "epilogue staging must fit in the operand ring");
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// one block load: 64 lanes x 16 bytes from sbase + voff (bytes) to LDS bytes [lds_addr, lds_addr + 1024).  No "memory"
// clobber: what orders these asynchronous LDS writes against the fragment reads is the vmcnt wait + barrier of the
// stage loop (both compiler barriers), never program order - and with the clobber the compiler kept every fragment
// read behind the load issued before it, one LDS latency per MFMA group.  volatile keeps the loads in order among
// themselves and against the waits.  m0 is written without telling the compiler (it rejects reserved registers in a clobber
// list): nothing else in this kernel uses it - no dynamically indexed register arrays, no LDS instruction that needs it.
__device__ __forceinline__ void frag_load(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr));
}
template <int N> __device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <typename DT, int ACT, int WC, int BK, int NS, int CT>
__global__ __launch_bounds__(256 * WC, (Geo<WC, BK, NS, CT>::WG_PER_CU)) void linear_ring_kernel(LinArgs a, int ncb, int nrb) {
    typedef Geo<WC, BK, NS, CT> G;
    constexpr int CW = G::CW;
    constexpr int BN = G::BN, NW = G::NW, KCH = G::KCH, RPL = G::RPL, LPR = G::LPR, XB = G::XB, STAGE_U4 = G::STAGE_U4;
    constexpr int NLX = G::NLX, NLW = G::NLW, NLD = G::NLD;
    extern __shared__ __attribute__((aligned(16))) u32x4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave & 3, wc = wave >> 2;                   // the wave's 64-row slab and column slab
    const int r16 = lane & 15, g = lane >> 4;
    // workgroup id -> (row block, column block): ids go round-robin over the 8 XCDs; inside an XCD consecutive
    // workgroups walk the column blocks of one row block
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int rb = (j / ncb) * 8 + xcd, cb = j % ncb;
    if (rb >= nrb) return;
    const int64_t row0 = (int64_t)rb * BM;
    const int col0 = cb * BN;
    const int K = a.K;
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    // loader: lane -> (row, k piece) inside each of its blocks; rows past the end re-read the last one
    const int lrow = lane / LPR, piece = (lane % LPR) ^ (BK == 32 ? (lrow >> 1) & 3 : lrow & 7);
    uint32_t voff[NLD];
#pragma unroll
    for (int i = 0; i < NLX; ++i) {
        int64_t r = row0 + RPL * (wave + NW * i) + lrow;
        r = r < a.rows ? r : a.rows - 1;
        voff[i] = (uint32_t)((r - row0) * a.ldx * 2 + piece * 16);
    }
#pragma unroll
    for (int i = 0; i < NLW; ++i) {
        int c = col0 + RPL * (wave + NW * i) + lrow;
        c = c < a.M ? c : a.M - 1;
        voff[NLX + i] = (uint32_t)((c - col0) * K * 2 + piece * 16);
    }
    const char* xs = reinterpret_cast<const char*>(a.x) + row0 * a.ldx * 2;       // scalar bases, advanced per step
    const char* ws = reinterpret_cast<const char*>(a.w) + (int64_t)col0 * K * 2;
    auto issue = [&](int slot) __attribute__((always_inline)) {
        const uint32_t sb = lds_base + slot * (STAGE_U4 * 16);
#pragma unroll
        for (int i = 0; i < NLX; ++i) frag_load(voff[i], xs, sb + (wave + NW * i) * 1024);
#pragma unroll
        for (int i = 0; i < NLW; ++i) frag_load(voff[NLX + i], ws, sb + (XB + wave + NW * i) * 1024);
        xs += 2 * BK; ws += 2 * BK;
    };
    // the same loads one at a time, for spreading over the MFMAs of a stage: issued in one burst after the barrier, the
    // 8 waves' loads queue behind each other in the CU's address unit and every wave stalls in its issue phase
    auto issue_one = [&](int slot, int idx) __attribute__((always_inline)) {
        const uint32_t sb = lds_base + slot * (STAGE_U4 * 16);
        if (idx < NLX) frag_load(voff[idx], xs, sb + (wave + NW * idx) * 1024);
        else frag_load(voff[idx], ws, sb + (XB + wave + NW * (idx - NLX)) * 1024);
        if (idx == NLD - 1) { xs += 2 * BK; ws += 2 * BK; }
    };

    f32x4 acc[CT][4];                              // [column tile][row tile]
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) acc[i][jj] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int nsteps = K / BK;
    // this lane's 16-byte slot for (16-row tile t, chunk c), relative to the stage: BK = 32: block t, slot
    // r16 * 4 + (g ^ swizzle); BK = 64: block 2 t + r16 / 8, slot (r16 % 8) * 8 + ((4 c + g) ^ (r16 % 8))
    auto rd = [&](int t, int c) __attribute__((always_inline)) {
        return BK == 32 ? t * 64 + r16 * 4 + (g ^ ((r16 >> 1) & 3))
                        : (2 * t + (r16 >> 3)) * 64 + (r16 & 7) * 8 + ((4 * c + g) ^ (r16 & 7));
    };
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) if (s < nsteps) issue(s);
    int slot = 0, fill = NS - 1;                                 // slot of step s; slot that step s + NS - 1 goes to
    // one stage: the fragment reads and MFMAs of slot `slot`, with the loads of stage s + NS - 1 spread over the
    // MFMA groups when MORE.  Two loops (main with loads, tail without) rather than a branch inside one: with the
    // branch the fragment reads were no longer issued ahead of the previous group's MFMAs.
#define RING_STAGE(MORE)                                                                                        \
    do {                                                                                                        \
        const u32x4* st = lds + slot * STAGE_U4;                                                                \
        _Pragma("unroll") for (int c = 0; c < KCH; ++c) {                                                       \
            s16x8 xf[4];                                                                                        \
            _Pragma("unroll") for (int jj = 0; jj < 4; ++jj) xf[jj] = __builtin_bit_cast(s16x8, st[rd(wr * 4 + jj, c)]); \
            _Pragma("unroll") for (int i = 0; i < CT; ++i) {                                                    \
                const s16x8 wf = __builtin_bit_cast(s16x8, st[XB * 64 + rd(wc * CT + i, c)]);                   \
                _Pragma("unroll") for (int jj = 0; jj < 4; ++jj) acc[i][jj] = DT::mfma32(wf, xf[jj], acc[i][jj]); \
                if (MORE && c * CT + i < NLD) issue_one(fill, c * CT + i);                                      \
            }                                                                                                   \
        }                                                                                                       \
        slot = slot + 1 == NS ? 0 : slot + 1;                                                                   \
        fill = fill + 1 == NS ? 0 : fill + 1;                                                                   \
    } while (0)
    int s = 0;
    for (; s + NS - 1 < nsteps; ++s) {
        wait_loads<NLD * (NS - 2)>();
        __syncthreads();                           // step s has landed for every wave; slot `fill` is no longer read
        RING_STAGE(true);
    }
    for (; s < nsteps; ++s) {
        if (s + NS - 2 < nsteps) wait_loads<NLD * (NS - 2)>(); else wait_loads<0>();
        __syncthreads();
        RING_STAGE(false);
    }
#undef RING_STAGE
    // epilogue.  After a transpose through LDS lane (rq, m) = (lane / 16, lane % 16) owns 8 consecutive columns
    // 8 m .. 8 m + 7 of rows rq + 4 q: 16 lanes write (and read the residual of) one 256-byte row segment.  The
    // residual (or, without one, the gate) for the whole 64 x 128 wave tile is requested up front, 16 loads in
    // flight, so that its latency is paid once per tile and not once per row group.
    const int m16 = lane & 15, rq = lane >> 4;
    const int colw = col0 + wc * CW + 8 * m16;                   // M % 8 == 0: the 8 columns are in or out together
    const bool col_ok = 8 * m16 < CW && colw < a.M;              // 96-column slabs leave lanes 12..15 of a row idle
    const u16* aux = static_cast<const u16*>(a.res ? a.res : a.gate);
    const int64_t ldaux = a.res ? a.ldr : a.ldgate;
    u32x4 pre[16];
    if (aux) {
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int64_t row = row0 + wr * 64 + (t >> 2) * 16 + rq + 4 * (t & 3);
            pre[t] = (u32x4){0u, 0u, 0u, 0u};
            if (col_ok && row < a.rows) pre[t] = *reinterpret_cast<const u32x4*>(aux + row * ldaux + colw);
        }
    }
    float bv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) bv[e] = 0.f;
    if (a.bias && col_ok) {
        const float4 b0 = *reinterpret_cast<const float4*>(a.bias + colw), b1 = *reinterpret_cast<const float4*>(a.bias + colw + 4);
        bv[0] = b0.x; bv[1] = b0.y; bv[2] = b0.z; bv[3] = b0.w; bv[4] = b1.x; bv[5] = b1.y; bv[6] = b1.z; bv[7] = b1.w;
    }
    __syncthreads();                               // operand ring dead: LDS becomes the staging area
    float* ep = reinterpret_cast<float*>(lds) + wave * (16 * EP_LD);          // private fp32 [16][128 + 4]
    u16* y = static_cast<u16*>(a.y);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
#pragma unroll
        for (int i = 0; i < CT; ++i)
            *reinterpret_cast<float4*>(ep + r16 * EP_LD + i * 16 + 4 * g) = make_float4(acc[i][jj][0], acc[i][jj][1], acc[i][jj][2], acc[i][jj][3]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int rl = rq + 4 * q;
            const int64_t row = row0 + wr * 64 + jj * 16 + rl;
            const float4 f0 = *reinterpret_cast<const float4*>(ep + rl * EP_LD + 8 * m16);
            const float4 f1 = *reinterpret_cast<const float4*>(ep + rl * EP_LD + 8 * m16 + 4);
            float v[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = keep_f32(apply_act16<ACT>(v[e] + bv[e]));
            const u32x4 p = pre[jj * 4 + q];
            if (a.res) {
#pragma unroll
                for (int e = 0; e < 4; ++e) { v[2 * e] += DT::to_f((u16)(p[e] & 0xffff)); v[2 * e + 1] += DT::to_f((u16)(p[e] >> 16)); }
            }
            if (a.gate && col_ok && row < a.rows) {
                const u32x4 gv = p;                    // residual and gate together are not taken (entry check)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (!(DT::to_f((u16)(gv[e] & 0xffff)) > 0.f)) v[2 * e] = 0.f;
                    if (!(DT::to_f((u16)(gv[e] >> 16)) > 0.f)) v[2 * e + 1] = 0.f;
                }
            }
            if (col_ok && row < a.rows) {
                u32x4 ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) ov[e] = DT::pack2(v[2 * e], v[2 * e + 1]);
                *reinterpret_cast<u32x4*>(y + lin_yoff(a, row) + colw) = ov;
            }
        }
    }
}

template <typename DT, int ACT, int WC, int BK, int NS, int CT>
bool launch_geo(const LinArgs& a, hipStream_t st) {
    typedef Geo<WC, BK, NS, CT> G;
    auto kern = linear_ring_kernel<DT, ACT, WC, BK, NS, CT>;
    static bool ready = false;                     // per instantiation; the attribute is process-wide per function
    if (!ready) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        ready = true;
    }
    const int64_t ncb = (a.M + G::BN - 1) / G::BN, nrb = (a.rows + BM - 1) / BM;
    const int64_t grid = 8 * ((nrb + 7) / 8) * ncb;
    if (grid > 0x7fffffffLL) return false;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(G::NT), G::LDS_BYTES, st, a, (int)ncb, (int)nrb);
    return true;
}

template <typename DT, int ACT>
bool launch_one(const LinArgs& a, hipStream_t st) {
    // 256-column tiles (half the operand traffic per MFMA) when the columns fill them
    if ((a.M % 256 == 0 || a.M >= 1024) && a.K % 64 == 0) return launch_geo<DT, ACT, 2, 64, 2, 8>(a, st);
    // 192-column tiles: one column block where 128-column tiles take two (the second half empty) and read x twice
    // (with more than one block of them and a short K the two-workgroups-per-CU narrow tiles win: 0.47 vs 0.51 ms
    // at K = M = 384, 786k rows; at K = 1536 it is 1.24 vs 1.14 the other way)
    if ((a.M == 192 || (a.M % 192 == 0 && a.M <= 768 && a.K >= 512)) && a.K % 64 == 0) return launch_geo<DT, ACT, 2, 64, 2, 6>(a, st);
    return launch_geo<DT, ACT, 1, 32, 3, 8>(a, st);
}

template <typename DT>
bool launch(const LinArgs& a, int act, hipStream_t st) {
    if (act == BSRL_ACT_RELU) return launch_one<DT, BSRL_ACT_RELU>(a, st);
    if (act == BSRL_ACT_GELU) return launch_one<DT, BSRL_ACT_GELU>(a, st);
    return launch_one<DT, BSRL_ACT_NONE>(a, st);
}

}  // namespace

bool bsrl_linear_ring(const LinArgs& a, int act, int dtype, hipStream_t st) {
    if (a.out_f32 || a.y2 || a.rows < 4096 || a.M % 8 != 0 || a.K % 32 != 0) return false;
    if (a.ldx % 8 != 0 || !bsrl_aligned(a.x, 16) || !bsrl_aligned(a.w, 16) || a.ldx > (1 << 22) || a.K > (1 << 22)) return false;
    if (a.ldy % 8 != 0 || a.y_gstride % 8 != 0 || !bsrl_aligned(a.y, 16) || (a.res && (a.ldr % 8 != 0 || !bsrl_aligned(a.res, 16)))) return false;
    // a load inside the row-group loop would put a vmcnt(0) wait there, and on this part that also waits for the
    // previous group's stores: residual and gate together go to the tiled kernel
    if (a.gate && (a.res || a.ldgate % 8 != 0 || !bsrl_aligned(a.gate, 16))) return false;
    return dtype == BSRL_F16 ? launch<F16>(a, act, st) : launch<BF16>(a, act, st);
}
