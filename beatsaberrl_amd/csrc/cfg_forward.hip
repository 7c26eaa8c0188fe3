// Whole config-model policy forward in ONE persistent kernel for gfx950.
//
// Shape class: T = 16 tokens per env, d = 128, 4 heads x 32, FFN multiple of 32,
// any number of layers, fp16 or bf16 operands with fp32 accumulate.
//
// Mapping.  One 16-row MFMA tile == one env (its 16 tokens).  A wave64 owns RT
// envs and carries their fp32 residual stream in registers for the whole
// forward (RT x 8 feature tiles x 4 VGPRs); LayerNorm, the QKV projection,
// attention (one 16x16x32 MFMA per head for the scores, softmax by two
// cross-lane butterflies, 16x16x16 MFMAs for P.V), the output projection, the
// FFN with its hidden kept in registers, and the 29x7 + 1 output projection
// all run wave-locally: activations never touch LDS or HBM.  The activation is
// always the MFMA operand whose free index is the TOKEN, so a GEMM's output
// fragment (4 consecutive features per lane) packs straight into the next
// GEMM's input fragment; the k order this implies (features 4g..4g+3 then
// 16+4g..16+4g+3 of each 32-chunk for lane group g) is baked into the weight
// image by bsrl_cfg_pack, so a weight fragment is one 16-byte LDS read per lane.
// The V projection swaps operand roles and so lands already transposed for P.V.
//
// Weights (~0.85 MB at 2 layers) stream from L2 in 8 KB stages (8 fragments) shared by the workgroup's 4 waves.
// Three pipelines, chosen on the host by shape and batch (same output bits):
//   * DMA  - the throughput forms' default: stages go straight from L2 into a 6-slot LDS ring
//            (global_load_lds_dwordx4), admitted in pairs: one vmcnt wait + barrier per two stages;
//   * RING - the latency form (B <= 4 per CU): the same transfers 13 stages ahead into a 14-slot ring, one env per wave;
//   * register-staged (models whose vectors + two rings overflow a CU's LDS): global loads three stages ahead into
//     registers, written to a 2-slot LDS ring one stage ahead, one barrier per stage.
// HBM traffic is the obs in, the logits out and, in the pruned form, each env's parked token-0 row (768 B).
//
// Final-block query pruning runs as ONE launch on the DMA pipeline (MERGE): every workgroup parks the token-0 rows of
// its own envs and, whenever 64 of them wait and once more at the end, switches its weight stream to the tail's stage
// range and runs the last block's output projection, FFN and the readout on them itself - no workgroup ever waits
// for another.  On the register-staged pipeline the tail is a second launch (MODE_TAIL).
//
// Replaces NotePolicy.forward_stacked (python/policy.py:1179-1344) for the
// benchmark-config model; the weight image is the analogue of the reference's
// flat fp16 replica buffer (python/fp16_linear.py:249-346).
#include "bsrl_common.h"
#include <mutex>
#include <type_traits>

namespace {

constexpr int D = 128;            // model width
constexpr int NT = D / 16;        // feature tiles
constexpr int KC = D / 32;        // 32-wide k chunks
constexpr int H = 4;              // heads (dh = 32)
constexpr int T = 16;             // tokens per env == MFMA tile rows
constexpr int STAGE_FRAGS = 8;
constexpr int STAGE_U4 = STAGE_FRAGS * 64;       // uint4 per stage (8 KB)
constexpr int EMB_STAGES = NT / 2;               // 4
constexpr int HEAD_TILES = 16;                   // 204 outputs padded to 256
constexpr int HEAD_STAGES = HEAD_TILES * KC / STAGE_FRAGS;   // 8

__host__ __device__ constexpr int layer_stages(int F) { return 3 * H + NT * KC / STAGE_FRAGS + 2 * (F / 32); }
__host__ __device__ constexpr int total_stages(int L, int F) { return EMB_STAGES + L * layer_stages(F) + HEAD_STAGES; }
// fp32 vector region (floats)
constexpr int V_BP = 0, V_BO = D, V_LAYER0 = 2 * D;
constexpr int LV_LN1G = 0, LV_LN1B = D, LV_BQ = 2 * D, LV_BK = 3 * D, LV_BV = 4 * D, LV_BOUT = 5 * D,
              LV_LN2G = 6 * D, LV_LN2B = 7 * D, LV_B1 = 8 * D;
__host__ __device__ constexpr int lv_b2(int F) { return 8 * D + F; }
__host__ __device__ constexpr int lv_size(int F) { return 9 * D + F; }
constexpr int FV_LNG = 0, FV_LNB = D, FV_BH = 2 * D, FV_SIZE = 2 * D + HEAD_TILES * 16;
__host__ __device__ constexpr int vec_floats(int L, int F) { return V_LAYER0 + L * lv_size(F) + FV_SIZE; }

struct FwdArgs {
    const uint4* frags; const float* vec;
    const void* obs; int64_t obs_ld; int obs_f32;
    int tok_vec;      // fp32 obs, 16-lane objects, 4-aligned proprio width and rows: the tokenizer reads 16-byte groups
    const int32_t* n_valid;
    float* logits; float* value;
    uint32_t* ws;
    const int4* pairs;            // PACK: tile -> the env that starts at rows 0 / 4 / 8 / 12 (-1: the slot continues the env
                                  // before it), written by cfg_pair_kernel
    const int32_t* n_packed;      // PACK: number of tiles in `pairs`
    int64_t B; int n_layers, F, s_begin, s_end, n_logits, final_ln, prop_dim, obj_dim;
    int t_begin, t_end;           // MERGE: stage range of the token-0 tail (the last block's output projection, FFN and the readout)
    int cus;          // CUs of the device (PACK: the remainder split below)
    int ring_epw;     // RING: envs per workgroup (1..4): one per wave, the other waves only feed the weight ring
};

// ---- helpers -------------------------------------------------------------------
template <typename DT> __device__ __forceinline__ uint32_t pack2(float a, float b) {
    return DT::pack2(a, b);
}
template <> __device__ __forceinline__ uint32_t pack2<F16>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<BF16>(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
union Frag8 { s16x8 v; uint32_t w[4]; uint4 u; };
union Frag4 { s16x4 v; uint32_t w[2]; };


// RING variant of the weight pipeline (the latency form): stages go global -> LDS directly (global_load_lds_dwordx4:
// one wave instruction lands one 1 KB fragment, lane l's 16 bytes at slot l), RING_DEPTH stages ahead of the one being
// consumed, into a ring of RING_DEPTH + 1 stage slots; no register staging, so the depth is bounded by LDS, not VGPRs.
// A lone workgroup walking ~100 stages is bound by the L2 round trip divided by the stages in flight: 3 in the
// register-staged pipeline, 13 here.
constexpr int RING_DEPTH = 13, RING_SLOTS = RING_DEPTH + 1;
// DMA variant (the throughput forms: whole forward / first launch): the same direct-to-LDS transfers into a ring of
// DMA_SLOTS stage slots, stages admitted in PAIRS - one vmcnt wait + barrier per two stages, then the two slots behind
// them are refilled - against one barrier, two LDS stores and two register-staged loads per stage in the
// register-staged pipeline.  While a pair is consumed, DMA_SLOTS - 4 further stages are in flight.
constexpr int DMA_SLOTS = 6, DMA_AHEAD = DMA_SLOTS - 4;
// m0 (the LDS base of the transfer) is written without telling the compiler, which rejects reserved registers in a
// clobber list: nothing else in these kernels uses it (no dynamically indexed register arrays, no instruction that
// reads m0).  No "memory" clobber: what orders the asynchronous LDS writes against the fragment reads is the explicit
// vmcnt wait + barrier of ring_advance.
__device__ __forceinline__ void ring_load(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr));
}
// two consecutive fragments: the instruction's immediate offset moves the global AND the LDS address, so the second
// transfer needs no second m0 write and no address arithmetic
__device__ __forceinline__ void ring_load2(uint32_t voff, const void* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024"
                 ::"v"(voff), "s"(sbase), "s"(lds_addr));
}

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Weight-stage pipeline: stage s lives in LDS slot s & 1; its global loads were issued 3
// stage-steps earlier into the register pair of the same parity (pr0a/pr0b or pr1a/pr1b).
// The four registers are plain named locals (never an indexed array: the prefetched data
// must stay in VGPRs while in flight, a stack slot would force a wait right after the load).
// ADVANCE_P(P): P = parity of the stage about to be consumed.
#define ADVANCE_P(P, RA, RB) do { \
        lds_barrier();                                   /* stage s complete in slot P; slot 1-P free */ \
        lds[1 - (P)][tid] = RA;                          /* stage s+1 -> slot 1-P */ \
        lds[1 - (P)][tid + 256] = RB; \
        const uint4* src_ = img + (int64_t)pnext * STAGE_U4 + tid;   /* stage s+3 -> the freed registers */ \
        RA = src_[0]; \
        RB = src_[256]; \
        pnext = pnext + 1 == a.s_end ? a.s_begin : pnext + 1; \
    } while (0)
// (RING: the advance happens inside the fragment fetch, one stage ahead - see ring_take)
// (DMA: the throughput forms' direct-to-LDS pipeline - see dma_advance)
#define ADVANCE(par) do { if (RING) { } else if (DMA) dma_advance(par); else if (par) ADVANCE_P(1, pr0a, pr0b); else ADVANCE_P(0, pr1a, pr1b); } while (0)
// TAIL launch: a workgroup streams its 44 stages for ONE tile with little arithmetic per stage, so the
// step time is the L2 latency of the weight stream divided by the stages in flight.  Four register
// sets (q0..q3) keep four stages in flight instead of two: ADVANCE4(Q), Q = index of the stage about to
// be consumed modulo 4, writes stage s+1 (set (Q+1) & 3) to the free slot and requests stage s+5 into it.
#define ADVANCE4(Q) do { \
        if ((Q) == 0) ADVANCE_P(0, q1a, q1b); else if ((Q) == 1) ADVANCE_P(1, q2a, q2b); \
        else if ((Q) == 2) ADVANCE_P(0, q3a, q3b); else ADVANCE_P(1, q0a, q0b); \
    } while (0)
// ADV(sidx): sidx = stage index counted from the start of the block (HEAD / FULL: only its parity
// matters) or from the start of the TAIL launch's own stage range (its value modulo 4 matters)
#define ADV(sidx) do { if (MODE == MODE_TAIL) ADVANCE4((sidx) & 3); else ADVANCE((sidx) & 1); } while (0)
#define WFRAG(par, f) (__builtin_bit_cast(s16x8, DMA ? ring[dma_cur * STAGE_U4 + (f) * 64 + lane] : lds[(RING || DMA) ? 0 : (par)][(RING || DMA) ? 0 : (f) * 64 + lane]))
// all 8 fragments of the current stage -> registers in one burst of LDS reads (one wait instead of 8)
#define LOAD_STAGE(par, W) s16x8 W[STAGE_FRAGS]; if (RING) ring_take(W); else _Pragma("unroll") for (int f_ = 0; f_ < STAGE_FRAGS; ++f_) W[f_] = WFRAG(par, f_)
// the same with the slot chosen at run time among the two (a wave-uniform value)
#define LOAD_STAGE_SLOT(slot, W) s16x8 W[STAGE_FRAGS]; if (RING) ring_take(W); else _Pragma("unroll") for (int f_ = 0; f_ < STAGE_FRAGS; ++f_) W[f_] = (slot) ? WFRAG(1, f_) : WFRAG(0, f_)

// MODE_FULL: the whole forward, one launch, every token of the last block computed.
// MODE_HEAD + MODE_TAIL: final-block query pruning (the reference's n_queries path,
//   python/policy.py:533-539: exact, because masking is key-side only).  HEAD runs the
//   tokenizer, blocks 0..L-2 and the last block's LN + QKV + attention, and parks the
//   token-0 row of every env (fp32 residual + attention-output fragments) in the
//   workspace; the tail re-tiles those rows 16 envs per MFMA tile and runs the last block's
//   output projection + FFN and the 29*K + 1 output projection on them - inside the HEAD
//   launch on the DMA pipeline (MERGE, below), as a launch of its own (MODE_TAIL) otherwise.
enum { MODE_FULL = 0, MODE_HEAD = 1, MODE_TAIL = 2 };
// Envs per 16-row MFMA tile in the TAIL launch.  Measured: 8 (twice the waves in flight, twice the weight stream)
// takes 30 us against 24 us with full tiles at B = 16384.
constexpr int TAIL_ENVS = 16;
// MERGE (the pruned form as ONE launch: every first launch on the direct-to-LDS pipeline): a workgroup runs the token-0
// tail of the envs it parked ITSELF - no other workgroup is ever waited for.  Their ids queue up in an LDS ring of
// TAIL_CAP entries; whenever a workgroup pass (4 waves x 16 envs) is full, and once more at the end for the rest,
// the weight stream switches to the tail's stage range for one pass.  A head pass parks at most 32 envs per
// workgroup (8 tiles x 4) onto fewer than 64 waiting ones, so 128 entries always suffice.
constexpr int TAIL_WG_ENVS = 4 * TAIL_ENVS, TAIL_CAP = 128;
constexpr int WS_DWORDS = 48;      // per (env, lane group): 32 fp32 residual + 16 dwords of attention output

// PACK (HEAD launch only): short envs share a 16-row tile under a block-diagonal key mask - two of at most 8 tokens
// (rows 0.. and 8..), four of at most 4 tokens (rows 0.., 4.., 8.., 12..), or one of at most 12 tokens with one of
// at most 4 behind it (rows 12..).  Every per-row computation (GEMMs,
// LayerNorm) is untouched by the row's position; the softmax sums and the P.V contraction see an env's keys a
// multiple of 4 lanes / k slots further on: a key's place inside its lane group of 4 is unchanged, whole groups move,
// and everything else a sum meets is an exact zero - an env's bits stay what they are alone in a tile.
// INK (a PACK + MERGE variant, batches of at most INK_MAX_ENVS): no tile table in memory and no table kernel before the
// launch.  Every workgroup classes the whole batch itself in its prologue (64 KB of key counts out of L2, beside the
// weight ring's first stages) and keeps, in LDS, a 2-bit class code per env and the four classes' exclusive prefixes
// over blocks of 64 envs; a tile's four slot entries are then SELECTED from those on the fly - lane i of the wave
// answers "which env is the r-th of class c" for slot i by a binary search over the prefixes and a rank select in the
// block's class mask - one pass ahead, while the pass's own observation loads are in flight.  The entries are
// those cfg_pair_kernel writes (same classes, same stable order, same tile order).
constexpr int INK_BLOCKS = 256, INK_MAX_ENVS = INK_BLOCKS * 64;
constexpr int INK_WORDS = INK_BLOCKS * 4 + 4 * INK_BLOCKS + 4;           // class bit planes, prefixes, totals (dwords)
constexpr size_t INK_BYTES = ((size_t)INK_WORDS * 4 + 255) & ~(size_t)255;
template <typename DT, int KRT, int ACT, int MODE, bool PACK = false, bool RING = false, bool DMA = false, bool INK = false>
__global__ __launch_bounds__(256, (KRT <= 2 && !RING) ? 2 : 1) void cfg_forward_kernel(FwdArgs a) {
    static_assert(!PACK || MODE == MODE_HEAD, "packing is a HEAD-launch variant");
    static_assert(!INK || (PACK && DMA && MODE == MODE_HEAD && KRT == 2), "the in-kernel tile table is a variant of the packed one-launch form");
    static_assert(!RING || MODE == MODE_FULL, "the ring pipeline is the one-launch latency form");
    static_assert(!DMA || (!RING && MODE != MODE_TAIL), "the paired direct-to-LDS pipeline serves the throughput forms");
    static_assert(KRT == 1 || KRT == 2, "the softmax butterflies pair the row tiles");
    constexpr bool MERGE = DMA && MODE == MODE_HEAD;
    __shared__ uint4 lds[(RING || DMA) ? 1 : 2][(RING || DMA) ? 64 : STAGE_U4];
    __shared__ int tail_list[MERGE ? TAIL_CAP : 1];   // MERGE: envs whose token-0 row this workgroup has parked, oldest first
    __shared__ int tail_wr;                           // MERGE: entries ever reserved in tail_list (monotonic)
    extern __shared__ float4 vlds4[];                 // every fp32 vector of the model, resident for the whole kernel
    const float* vlds = reinterpret_cast<const float*>(vlds4);
    // RING: the stage ring sits behind the vectors (1 KB aligned) in the dynamic region
    const int ring_off_u4 = (vec_floats(a.n_layers, a.F) / 4 + 63) & ~63;
    const uint4* ring = reinterpret_cast<const uint4*>(vlds4) + ring_off_u4;
    int ring_cur = RING_SLOTS - 1;                    // slot of the stage last consumed (the first advance wraps to 0)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const float scale_l2e = 0.17677669529663688110f * 1.44269504088896340736f;      // log2(e) / sqrt(32)
    constexpr int ENVS_PER_TILE = MODE == MODE_TAIL ? TAIL_ENVS : 1;     // envs per 16-row MFMA tile
    constexpr int ENVS_PER_WG = 4 * KRT * ENVS_PER_TILE;
    // PACK: the tile count, written by the table kernel just before this launch (on whichever XCD ran it: a fabric round
    // trip of ~2 us from here).  Requested first thing, consumed behind the prologue, which takes about as long.
    int np_raw = 0;
    if (PACK && !INK) asm volatile("global_load_dword %0, %1, off" : "=v"(np_raw) : "v"(a.n_packed));

    const uint4* img = a.frags;
    const uint32_t ring_base = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)const_cast<uint4*>(ring);
    const int uwave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint4 pr0a, pr0b, pr1a, pr1b;
    uint4 q0a, q0b, q1a, q1b, q2a, q2b, q3a, q3b;       // TAIL launch only
    int pnext;
    // RING: this wave's two fragments of stage `stage` -> ring slot `slot` (every wave loads, working or not: leaving the
    // loads to the waves without an env - 3 + 3 + 2 fragments - measured slower, 36 against 33 us per forward)
    // The transfers address the image and the ring by running BYTE offsets (a stage and a slot are both 8 KB): one
    // 64-bit scalar add per issue instead of two multiplies per index.
    constexpr uint32_t STAGE_B = STAGE_U4 * 16;
    const char* wsrc = reinterpret_cast<const char*>(img) + uwave * 2048;      // this wave's two fragments of a stage
    const uint32_t wdst = ring_base + uwave * 2048;
    uint32_t src_off = 0;                             // byte offset of stage pnext
    const uint32_t src_begin = (uint32_t)a.s_begin * STAGE_B, src_end = (uint32_t)a.s_end * STAGE_B;
    // The stage sequence is a chain of segments (stage ranges).  seg_end closes the segment being fetched; the one
    // after it is (nxt_begin, nxt_end).  Without MERGE there is one range, walked cyclically.  MERGE: the consumer
    // names the successor at the start of every segment - the fetch runs at most DMA_SLOTS stages ahead of it and
    // every segment is longer, so the successor is always known before the fetch reaches a segment's end.
    const uint32_t tail_begin = (uint32_t)a.t_begin * STAGE_B, tail_end = (uint32_t)a.t_end * STAGE_B;
    uint32_t seg_end = src_end, nxt_begin = src_begin, nxt_end = src_end;
    auto ring_issue_off = [&](uint32_t slot_off) __attribute__((always_inline)) {     // stage pnext -> the slot at slot_off
        ring_load2(lane * 16, wsrc + src_off, wdst + slot_off);
        src_off += STAGE_B;
        if (MERGE) { if (src_off == seg_end) { src_off = nxt_begin; seg_end = nxt_end; } }
        else src_off = src_off == src_end ? src_begin : src_off;
    };
    // MERGE bookkeeping, all wave-uniform: t_rd = entries of tail_list consumed so far (monotonic), t_cnt = entries
    // waiting as of the last decision, t_more_head = another head-type pass of this workgroup follows the current one
    // (set by the pass loop), t_tail_next = the segment after the current one is a tail pass
    int t_rd = 0, t_cnt = 0;
    bool t_more_head = false, t_tail_next = false;
    // RING: called when the next stage is about to be consumed; on return it is readable in slot ring_cur
    uint32_t ring_off = (RING_SLOTS - 1) * STAGE_B;   // byte offset of slot ring_cur
    auto ring_advance = [&]() __attribute__((always_inline)) {
        const uint32_t freed = ring_off;              // the slot of the stage consumed last
        ring_cur = ring_cur + 1 == RING_SLOTS ? 0 : ring_cur + 1;
        ring_off = ring_off + STAGE_B == RING_SLOTS * STAGE_B ? 0 : ring_off + STAGE_B;
        // this wave's loads of that stage have landed once at most the RING_DEPTH - 1 younger stages' are outstanding
        // (loads retire in order; any other load or store in flight only makes the wait stricter) ...
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (RING_DEPTH - 1)) : "memory");
        lds_barrier();                                // ... and every wave's have; every wave is done reading the stage before
        ring_issue_off(freed);                        // its slot takes the stage RING_DEPTH ahead
    };
    // DMA: entry of the next stage (par = its parity in the launch's stage range): on return it is readable in slot
    // dma_cur.  An even stage admits itself and its successor: this wave's loads of both have landed once at most the
    // DMA_AHEAD younger stages' are outstanding, the barrier says the same of every wave's and that every wave is done
    // reading the two stages before; their slots take the next two stages.
    int dma_cur = DMA_SLOTS - 1;
    uint32_t dma_off = (DMA_SLOTS - 1) * STAGE_B, dma_prev = (DMA_SLOTS - 2) * STAGE_B;     // byte offsets of slot dma_cur and the one before
    auto dma_advance = [&](int par) __attribute__((always_inline)) {
        const uint32_t older = dma_prev;
        dma_prev = dma_off;
        dma_cur = dma_cur + 1 == DMA_SLOTS ? 0 : dma_cur + 1;
        dma_off = dma_off + STAGE_B == DMA_SLOTS * STAGE_B ? 0 : dma_off + STAGE_B;
        if (par == 0) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * DMA_AHEAD) : "memory");
            lds_barrier();
            ring_issue_off(older);                    // the two slots behind the pair being admitted
            ring_issue_off(dma_prev);
        }
    };
    // RING: the working waves keep the NEXT stage's eight fragments in registers (wnext), fetched from LDS while the
    // current stage is being computed: a lone working wave would otherwise sit out one LDS round trip per stage
    // (~100 stages per forward) with nothing else to run.  ring_take hands out the fragments of the stage about to be
    // computed, advances the ring and requests the stage after it.  The LDS reads are asm so that they are issued HERE
    // (the compiler would sink plain loads to their use); the lgkmcnt wait that makes them usable carries wnext as an
    // operand so that no use of it can be scheduled above the wait.
    s16x8 wnext[RING ? STAGE_FRAGS : 1];
    auto ring_fetch = [&]() __attribute__((always_inline)) {
        const uint32_t addr = ring_base + ring_off + lane * 16;
#pragma unroll
        for (int f = 0; f < STAGE_FRAGS; ++f)
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(wnext[RING ? f : 0]) : "v"(addr), "n"(f * 1024));
    };
    auto ring_take = [&](s16x8 (&W)[STAGE_FRAGS]) __attribute__((always_inline)) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wnext[0]), "+v"(wnext[RING ? 1 : 0]), "+v"(wnext[RING ? 2 : 0]), "+v"(wnext[RING ? 3 : 0]),
                       "+v"(wnext[RING ? 4 : 0]), "+v"(wnext[RING ? 5 : 0]), "+v"(wnext[RING ? 6 : 0]), "+v"(wnext[RING ? 7 : 0])
                     :: "memory");
#pragma unroll
        for (int f = 0; f < STAGE_FRAGS; ++f) W[f] = wnext[RING ? f : 0];
        ring_advance();
        ring_fetch();
    };
    if (RING) {
        // prologue: RING_DEPTH stages in flight (the weight image holds at least that many), then the vectors
        src_off = src_begin;
#pragma unroll
        for (int i = 0; i < RING_DEPTH; ++i) ring_issue_off(i * STAGE_B);
        const int nv4 = vec_floats(a.n_layers, a.F) / 4;
        for (int i = tid; i < nv4; i += 256) vlds4[i] = reinterpret_cast<const float4*>(a.vec)[i];
        lds_barrier();
        ring_advance();             // the first stage is readable ...
        ring_fetch();               // ... and on its way to registers (every wave: the waves without an env never wait for it)
    } else if (DMA) {
        // prologue: DMA_SLOTS - 2 stages in flight (every launch's stage range is longer and even), then the vectors
        src_off = src_begin;
#pragma unroll
        for (int i = 0; i < DMA_SLOTS - 2; ++i) ring_issue_off(i * STAGE_B);
        const int nv4 = vec_floats(a.n_layers, a.F) / 4;
        for (int i = tid; i < nv4; i += 256) vlds4[i] = reinterpret_cast<const float4*>(a.vec)[i];
        if (tid == 0) tail_wr = 0;
        lds_barrier();
    } else {   // prologue: first stage -> LDS slot 0; the next two (TAIL: four) in flight (stage counts per mode are even)
        const int s0 = a.s_begin;
        const uint4 s0a = img[(int64_t)s0 * STAGE_U4 + tid], s0b = img[(int64_t)s0 * STAGE_U4 + tid + 256];
        if (MODE == MODE_TAIL) {
            q1a = img[(int64_t)(s0 + 1) * STAGE_U4 + tid]; q1b = img[(int64_t)(s0 + 1) * STAGE_U4 + tid + 256];
            q2a = img[(int64_t)(s0 + 2) * STAGE_U4 + tid]; q2b = img[(int64_t)(s0 + 2) * STAGE_U4 + tid + 256];
            q3a = img[(int64_t)(s0 + 3) * STAGE_U4 + tid]; q3b = img[(int64_t)(s0 + 3) * STAGE_U4 + tid + 256];
            q0a = img[(int64_t)(s0 + 4) * STAGE_U4 + tid]; q0b = img[(int64_t)(s0 + 4) * STAGE_U4 + tid + 256];
        } else {
            pr1a = img[(int64_t)(s0 + 1) * STAGE_U4 + tid]; pr1b = img[(int64_t)(s0 + 1) * STAGE_U4 + tid + 256];
        }
        lds[0][tid] = s0a; lds[0][tid + 256] = s0b;
        if (MODE != MODE_TAIL) { pr0a = img[(int64_t)(s0 + 2) * STAGE_U4 + tid]; pr0b = img[(int64_t)(s0 + 2) * STAGE_U4 + tid + 256]; }
        constexpr int AHEAD = MODE == MODE_TAIL ? 5 : 3;
        pnext = s0 + AHEAD >= a.s_end ? a.s_begin + (s0 + AHEAD - a.s_end) : s0 + AHEAD;
        // No global load other than the weight pipeline may sit in the steady state: vmcnt retires
        // in order, so waiting on a late bias load would also drain the prefetches issued before it.
        const int nv4 = vec_floats(a.n_layers, a.F) / 4;
        for (int i = tid; i < nv4; i += 256) vlds4[i] = reinterpret_cast<const float4*>(a.vec)[i];
        lds_barrier();
    }

    if (PACK && !INK) asm volatile("s_waitcnt vmcnt(0)" : "+v"(np_raw) :: "memory");
    // INK: class codes and prefixes of the whole batch -> LDS (behind the ring).  Classes as cfg_pair_kernel's: by key
    // count n_valid >> 2 = 0 tiny, 1 mid, 2 host, 3 (or more, or negative) long; envs past the batch's end count as long
    // ones behind every real env, which no select ever reaches.
    uint32_t* const ink_code = reinterpret_cast<uint32_t*>(const_cast<uint4*>(ring) + DMA_SLOTS * STAGE_U4);   // [block][4]: 2 bits per env
    uint32_t* const ink_pf = ink_code + INK_BLOCKS * 4;                                                       // [class][block]
    uint32_t* const ink_tot = ink_pf + 4 * INK_BLOCKS;                                                        // [class]
    int ink_tt = 0, ink_tm = 0, ink_th = 0, ink_first_quad = 0, ink_first_host = 0, ink_first_long = 0;
    if constexpr (INK) {
        // wave w classes envs [4096 w, 4096 w + 4096): sixteen coalesced 16-byte loads per lane, all in flight at once
        // (one memory round trip), the four 2-bit codes of a load written as ONE byte into the code array - which is
        // thereby in env order, 16 envs to a dword -, then lane l reads back block 64 w + l whole and counts its classes
        const int nB = (int)a.B, nq_full = nB >> 2;                        // whole groups of four envs
        const int4* nvq = reinterpret_cast<const int4*>(a.n_valid);        // 16-byte aligned (a condition of packing)
        uint32_t tail_byte = 0xFFu;                                        // the codes of the last B % 4 envs (then ghosts)
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int e = nq_full * 4 + k;
            const uint32_t c = (uint32_t)a.n_valid[e < nB ? e : nB - 1] >> 2;
            const uint32_t code = (e < nB && c < 3u) ? c : 3u;
            tail_byte = (tail_byte & ~(3u << (2 * k))) | (code << (2 * k));
        }
        int4 v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = make_int4(0, 0, 0, 0);
        if (nq_full > 0) {
#pragma unroll
            for (int i = 0; i < 16; ++i) { const int q = (uwave * 16 + i) * 64 + lane; v[i] = nvq[q < nq_full ? q : nq_full - 1]; }
        }
        unsigned char* const cbytes = reinterpret_cast<unsigned char*>(ink_code);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int q = (uwave * 16 + i) * 64 + lane;
            auto c2 = [](int nv) __attribute__((always_inline)) { const uint32_t c = (uint32_t)nv >> 2; return c < 3u ? c : 3u; };
            uint32_t byte = c2(v[i].x) | (c2(v[i].y) << 2) | (c2(v[i].z) << 4) | (c2(v[i].w) << 6);
            byte = q < nq_full ? byte : q == nq_full ? tail_byte : 0xFFu;
            cbytes[q] = (unsigned char)byte;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                 // the wave's own bytes (the LDS serves a wave in order)
        const int blk = uwave * 64 + lane;
        const uint4 cw = reinterpret_cast<const uint4*>(ink_code)[blk];
        const uint32_t cwd[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t n = 0;
#pragma unroll
            for (int d = 0; d < 4; ++d) { const uint32_t x = cwd[d] ^ (0x55555555u * c); n += __popc(~(x | (x >> 1)) & 0x55555555u); }
            ink_pf[c * INK_BLOCKS + blk] = n;
        }
        lds_barrier();
        if (uwave == 0) {                                                  // counts -> exclusive prefixes, 4 blocks to a lane
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint4* row = reinterpret_cast<uint4*>(ink_pf + c * INK_BLOCKS);
                const uint4 v = row[lane];
                const uint32_t sum = v.x + v.y + v.z + v.w;
                uint32_t incl = sum;
#pragma unroll
                for (int d = 1; d < WAVE; d <<= 1) { const uint32_t up = __shfl_up(incl, d, WAVE); if (lane >= d) incl += up; }
                const uint32_t ex = incl - sum;
                row[lane] = make_uint4(ex, ex + v.x, ex + v.x + v.y, ex + v.x + v.y + v.z);
                if (lane == WAVE - 1) ink_tot[c] = incl;
            }
        }
        lds_barrier();
        ink_tt = __builtin_amdgcn_readfirstlane((int)ink_tot[0]);
        ink_tm = __builtin_amdgcn_readfirstlane((int)ink_tot[1]);
        ink_th = __builtin_amdgcn_readfirstlane((int)ink_tot[2]);
        const int loose = ink_tt > ink_th ? ink_tt - ink_th : 0;           // tiny envs without a host
        ink_first_quad = (ink_tm + 1) / 2;
        ink_first_host = ink_first_quad + (loose + 3) / 4;
        ink_first_long = ink_first_host + ink_th;
    }
    // INK: the four slot entries of the KRT consecutive tiles from t0 on (t0 the same in every lane), as cfg_pair_kernel
    // would have written them: lane 4 rt + s answers for slot s of tile t0 + rt, the answers go to out[rt][s]
    auto ink_entries = [&](const int t0, int (&out)[PACK ? KRT : 1][4]) __attribute__((always_inline)) {
        const int n_all = ink_first_long + ((int)a.B - ink_tt - ink_tm - ink_th);
        int t = t0 + ((lane >> 2) & (KRT - 1));
        t = t < n_all ? t : n_all - 1;
        const int sl = lane & 3;
        int cls, rank; bool on;
        if (t < ink_first_quad) { cls = 1; rank = 2 * t + (sl >> 1); on = (sl & 1) == 0 && rank < ink_tm; }
        else if (t < ink_first_host) { cls = 0; rank = ink_th + 4 * (t - ink_first_quad) + sl; on = rank < ink_tt; }
        else if (t < ink_first_long) { cls = sl == 3 ? 0 : 2; rank = t - ink_first_host; on = sl == 0 || (sl == 3 && rank < ink_tt); }
        else { cls = 3; rank = t - ink_first_long; on = sl == 0; }
        rank = on ? rank : 0;
        const uint32_t* pf = ink_pf + cls * INK_BLOCKS;
        int j = 0;                                                         // the last block that starts at or before the rank
#pragma unroll
        for (int step = INK_BLOCKS / 2; step > 0; step >>= 1) j += pf[j + step] <= (uint32_t)rank ? step : 0;
        const uint32_t rr = (uint32_t)rank - pf[j];
        // the block's codes (16 envs to a dword, 2 bits each) -> one bit per env of the class, at the even positions
        const uint4 cw = reinterpret_cast<const uint4*>(ink_code)[j];
        const uint32_t pat = 0x55555555u * (uint32_t)cls;
        auto mask_of = [&](uint32_t w) __attribute__((always_inline)) { const uint32_t x = w ^ pat; return ~(x | (x >> 1)) & 0x55555555u; };
        const uint32_t m0 = mask_of(cw.x), m1 = mask_of(cw.y), m2 = mask_of(cw.z), m3 = mask_of(cw.w);
        const uint32_t s1 = __popc(m0), s2 = s1 + __popc(m1), s3 = s2 + __popc(m2);
        const int dw = (rr >= s1 ? 1 : 0) + (rr >= s2 ? 1 : 0) + (rr >= s3 ? 1 : 0);
        const uint32_t w = dw == 0 ? m0 : dw == 1 ? m1 : dw == 2 ? m2 : m3;
        const uint32_t r2 = rr - (dw == 0 ? 0u : dw == 1 ? s1 : dw == 2 ? s2 : s3);
        int pos = 0;                                                       // the r2-th set bit of w: the most bits below it that hold at most r2 ones
#pragma unroll
        for (int step = 16; step > 0; step >>= 1) pos += (uint32_t)__popc(w & ((1u << (pos + step)) - 1u)) <= r2 ? step : 0;
        const int env = on ? j * 64 + dw * 16 + (pos >> 1) : -1;
#pragma unroll
        for (int rt = 0; rt < (PACK ? KRT : 1); ++rt)
#pragma unroll
            for (int i = 0; i < 4; ++i) out[rt][i] = __builtin_amdgcn_readlane(env, rt * 4 + i);
    };
    // 16-row tiles (PACK) or envs to cover; the loaded count is the same in every lane, and said to be so: the pass loop
    // and (MERGE) the stage-fetch addresses derived from it must stay in scalar registers
    const int64_t n_units = INK ? (int64_t)(ink_first_long + ((int)a.B - ink_tt - ink_tm - ink_th))
                                : PACK ? (int64_t)__builtin_amdgcn_readfirstlane(np_raw) : a.B;
    const int64_t ntiles = RING ? (a.B + a.ring_epw - 1) / a.ring_epw : (n_units + ENVS_PER_WG - 1) / ENVS_PER_WG;

    // One pass of this wave over the weight stream with RT row tiles.  A generic lambda so that the packed first launch
    // can hold two bodies: two row tiles per wave for the bulk, ONE for the remainder tiles of the last round (below).
    // env0: the wave's first env (or first tile, PACK).
    // PACK: the table entries of the wave's NEXT pass ride along with this pass's own input loads (one wait for both) and
    // stay in scalar registers, so that a pass starts its key-count and observation loads without first waiting for
    // its table entries (one L2 round trip per pass).  next_wg0 = the first tile of the WORKGROUP's next bulk pass (the
    // same in every wave, and visibly so to the compiler: what hangs on it must stay wave-uniform), < 0: none.
    int pre_pr[PACK ? KRT : 1][4];
    bool have_pre = false;
    // tail_tag (MERGE): this pass is a token-0 tail pass of the workgroup's own parked envs, on the tail's stage range
    auto pass = [&](auto rt_tag, auto tail_tag, const int64_t env0, const int64_t next_wg0) __attribute__((always_inline)) {
        constexpr int RT = decltype(rt_tag)::value;
        constexpr bool TAILP = MODE == MODE_TAIL || decltype(tail_tag)::value;     // rows are envs (token 0 of each)
        static_assert(!decltype(tail_tag)::value || (MERGE && RT == 1), "merged tail passes run one row tile per wave");
        // MERGE: called right behind the first stage admission of a segment (its barrier has made every wave's
        // reservations for this pass visible): what follows this segment?
        auto merge_decide = [&]() __attribute__((always_inline)) {
            if (!MERGE) return;
            if (!decltype(tail_tag)::value) {
                const int wr = __builtin_amdgcn_readfirstlane(__hip_atomic_load(&tail_wr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
                t_cnt = wr - t_rd;
                t_tail_next = t_cnt >= TAIL_WG_ENVS || (!t_more_head && t_cnt > 0);
            }
            nxt_begin = t_tail_next ? tail_begin : src_begin;
            nxt_end = t_tail_next ? tail_end : src_end;
        };
        // every lambda below is force-inlined: one left out of line would take the residual registers by reference,
        // i.e. through scratch memory (seen with the bf16 instantiations, whose pack helper is larger)
        float kmask[RT][4];     // additive key mask for keys 4g..4g+3 of each env: 0 (attendable) or -inf
        f32x4 x[RT][NT];
        Frag8 hf[RT][KC];       // LayerNorm output as GEMM operand fragments
        Frag8 of[RT][KC];       // attention output fragments (chunk == head)

        // y = LN(x) * gamma + beta (or the raw x when !affine), packed as operand fragments
        auto norm_to_frags = [&](const float* gptr, const float* bptr, bool normalise, Frag8 (&dst)[RT][KC]) __attribute__((always_inline)) {
            float4 gm[NT], bt[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                gm[nt] = make_float4(1.f, 1.f, 1.f, 1.f); bt[nt] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (normalise) {
                    gm[nt] = *reinterpret_cast<const float4*>(gptr + 16 * nt + 4 * g);
                    bt[nt] = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
                }
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                float mean = 0.f, rstd = 1.f;
                if (normalise) {
                    // one pass: var = E[x^2] - mean^2, clamped at 0 (the reference kernel's formula,
                    // python/beat_arena_env/csrc/layer_norm.cu:14-21); both sums ride one butterfly
                    float s = 0.f, q = 0.f;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) { s += x[rt][nt][i]; q = fmaf(x[rt][nt][i], x[rt][nt][i], q); }
                    rows_reduce2(s, q, OpAdd());
                    mean = s * (1.0f / D);
                    rstd = rsqrtf(fmaxf(fmaf(-mean, mean, q * (1.0f / D)), 0.f) + 1e-5f);
                }
                const float shift = -mean * rstd;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    // (x - mean) * rstd as one fma, then the affine
                    const float y0 = fmaf(fmaf(x[rt][nt][0], rstd, shift), gm[nt].x, bt[nt].x);
                    const float y1 = fmaf(fmaf(x[rt][nt][1], rstd, shift), gm[nt].y, bt[nt].y);
                    const float y2 = fmaf(fmaf(x[rt][nt][2], rstd, shift), gm[nt].z, bt[nt].z);
                    const float y3 = fmaf(fmaf(x[rt][nt][3], rstd, shift), gm[nt].w, bt[nt].w);
                    dst[rt][nt >> 1].w[(nt & 1) * 2] = pack2<DT>(y0, y1);
                    dst[rt][nt >> 1].w[(nt & 1) * 2 + 1] = pack2<DT>(y2, y3);
                }
            }
        };
        auto add_bias = [&](const float* bptr) __attribute__((always_inline)) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 b = *reinterpret_cast<const float4*>(bptr + 16 * nt + 4 * g);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) { x[rt][nt][0] += b.x; x[rt][nt][1] += b.y; x[rt][nt][2] += b.z; x[rt][nt][3] += b.w; }
            }
        };

        // ---- LN1 + QKV + attention of one block (12 stages), head by head: fills `of` ----
        auto attention = [&](const float* lv) __attribute__((always_inline)) {
            norm_to_frags(lv + LV_LN1G, lv + LV_LN1B, true, hf);
#pragma unroll
            for (int hd = 0; hd < H; ++hd) {
                Frag8 qf[RT], kf[RT];
                Frag4 vt[RT][2];
#pragma unroll
                for (int part = 0; part < 3; ++part) {
                    const int par = (hd * 3 + part) & 1;        // stage parity (the block starts on an even stage)
                    ADVANCE(par);
                    LOAD_STAGE(par, wf);
                    f32x4 acc[2][RT];
#pragma unroll
                    for (int ntl = 0; ntl < 2; ++ntl) {
                        float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (part < 2) b = *reinterpret_cast<const float4*>(lv + (part == 0 ? LV_BQ : LV_BK) + 32 * hd + 16 * ntl + 4 * g);
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt) acc[ntl][rt] = (f32x4){b.x, b.y, b.z, b.w};
                    }
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                            for (int rt = 0; rt < RT; ++rt) {
                                const s16x8 w = wf[ntl * KC + c];
                                if (part < 2) acc[ntl][rt] = DT::mfma32(w, hf[rt][c].v, acc[ntl][rt]);
                                else acc[ntl][rt] = DT::mfma32(hf[rt][c].v, w, acc[ntl][rt]);   // V^T: roles swapped
                            }
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                        for (int ntl = 0; ntl < 2; ++ntl) {
                            const uint32_t lo = pack2<DT>(acc[ntl][rt][0], acc[ntl][rt][1]);
                            const uint32_t hi = pack2<DT>(acc[ntl][rt][2], acc[ntl][rt][3]);
                            if (part == 0) { qf[rt].w[ntl * 2] = lo; qf[rt].w[ntl * 2 + 1] = hi; }
                            else if (part == 1) { kf[rt].w[ntl * 2] = lo; kf[rt].w[ntl * 2 + 1] = hi; }
                            else { vt[rt][ntl].w[0] = lo; vt[rt][ntl].w[1] = hi; }
                        }
                }
                // scores^T = K Q^T (lane: query r16, keys 4g..4g+3), softmax over keys, O = P V (+ b_v)
                const float4 bv0 = *reinterpret_cast<const float4*>(lv + LV_BV + 32 * hd + 4 * g);
                const float4 bv1 = *reinterpret_cast<const float4*>(lv + LV_BV + 32 * hd + 16 + 4 * g);
                // both row tiles side by side: their max / sum butterflies share the row exchanges
                float sv[RT][4], mx[2], sm[2];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const f32x4 sc = DT::mfma32(kf[rt].v, qf[rt].v, (f32x4){0.f, 0.f, 0.f, 0.f});
                    // raw scores + additive key mask (0 / -inf); softmax of (scale * s) = exp2((s - max) * scale*log2e)
#pragma unroll
                    for (int i = 0; i < 4; ++i) sv[rt][i] = sc[i] + kmask[rt][i];
                    mx[rt] = fmaxf(fmaxf(sv[rt][0], sv[rt][1]), fmaxf(sv[rt][2], sv[rt][3]));
                }
                if (RT == 1) mx[1] = mx[0];
                rows_reduce2(mx[0], mx[1], OpMax());
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const float ms = -mx[rt] * scale_l2e;
                    sm[rt] = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) { sv[rt][i] = __builtin_amdgcn_exp2f(fmaf(sv[rt][i], scale_l2e, ms)); sm[rt] += sv[rt][i]; }
                }
                if (RT == 1) sm[1] = sm[0];
                rows_reduce2(sm[0], sm[1], OpAdd());
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const float inv = __builtin_amdgcn_rcpf(sm[rt]);
                    Frag4 pf;
                    pf.w[0] = pack2<DT>(sv[rt][0] * inv, sv[rt][1] * inv);
                    pf.w[1] = pack2<DT>(sv[rt][2] * inv, sv[rt][3] * inv);
                    const f32x4 o0 = DT::mfma16(vt[rt][0].v, pf.v, (f32x4){bv0.x, bv0.y, bv0.z, bv0.w});
                    const f32x4 o1 = DT::mfma16(vt[rt][1].v, pf.v, (f32x4){bv1.x, bv1.y, bv1.z, bv1.w});
                    of[rt][hd].w[0] = pack2<DT>(o0[0], o0[1]); of[rt][hd].w[1] = pack2<DT>(o0[2], o0[3]);
                    of[rt][hd].w[2] = pack2<DT>(o1[0], o1[1]); of[rt][hd].w[3] = pack2<DT>(o1[2], o1[3]);
                }
            }
        };

        // ---- output projection onto the residual (4 stages), then LN2 + FFN (2 * F/32 stages) ----
        auto proj_and_ffn = [&](const float* lv) __attribute__((always_inline)) {
            add_bias(lv + LV_BOUT);
#pragma unroll
            for (int st = 0; st < NT / 2; ++st) {
                ADV(st);                    // 12 stages precede in the block (parity restarts even); TAIL starts here
                if (decltype(tail_tag)::value && st == 0) merge_decide();
                LOAD_STAGE(st & 1, wf);
#pragma unroll
                for (int c = 0; c < KC; ++c)
#pragma unroll
                    for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt) x[rt][2 * st + ntl] = DT::mfma32(wf[ntl * KC + c], of[rt][c].v, x[rt][2 * st + ntl]);
            }
            norm_to_frags(lv + LV_LN2G, lv + LV_LN2B, true, hf);
            add_bias(lv + lv_b2(a.F));
            // Software-pipelined over 32-wide hidden chunks.  MFMA and VALU work only overlap when they
            // alternate finely inside one wave (measured on gfx950: 2 waves per SIMD running an MFMA
            // phase and a VALU phase side by side take the SUM of the two), so every phase pairs 8*RT
            // MFMAs with half a chunk of activation work, pinned two MFMAs + one activation at a time:
            //   phase 1 (stage W1(ch+1)): up-projection of chunk ch+1  ||  activation of chunk ch, upper row tiles
            //   phase 2 (stage W2(ch))  : down-projection of chunk ch  ||  activation of chunk ch+1, lower row tiles
            // Stage order in the image: W1(0), {W1(ch+1), W2(ch)}..., W2(last).
            const int nch = a.F / 32;
            constexpr int RH = RT / 2;                  // row tiles per activation half (RT == 1: no split)
            f32x4 accA[2][RT];
            Frag8 hidA[RT];                             // activation of the current chunk, as operand fragments
            auto up_init = [&](int ch, f32x4 (&acc)[2][RT]) __attribute__((always_inline)) {
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const float4 b = *reinterpret_cast<const float4*>(lv + LV_B1 + 32 * ch + 16 * ntl + 4 * g);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[ntl][rt] = (f32x4){b.x, b.y, b.z, b.w};
                }
            };
            // activation of one (row tile, n-tile) accumulator = 4 hidden units -> 2 packed dwords
            auto act4 = [&](const f32x4& v, Frag8& dst, int ntl) __attribute__((always_inline)) {
                dst.w[ntl * 2] = pack2<DT>(apply_act16<ACT>(v[0]), apply_act16<ACT>(v[1]));
                dst.w[ntl * 2 + 1] = pack2<DT>(apply_act16<ACT>(v[2]), apply_act16<ACT>(v[3]));
            };
            if (RT == 1) {
                // Single row tile (TAIL launch): plain chunk loop, no split.  Stage indices count from the TAIL launch's
                // first stage: 0..3 the output projection, 4 = W1(0), then W1(ch+1) = 5 + 2 ch and W2(ch) = 6 + 2 ch, the
                // last W2 = 3 + 2 nch.  The hidden width is a multiple of 64 (nch even), and a loop trip advances two
                // chunks = four stages, so every stage keeps its place in the rotation of the four prefetch register sets.
                // The loop body is branch-free on purpose: with the last chunk's stage under a condition inside it, the
                // compiler could no longer count the loads in flight at the loop head and drained the whole prefetch queue
                // (s_waitcnt vmcnt(0)) before every stage - one L2 round trip per stage, 32 times per tile.
                auto up = [&](int ch, int slot) __attribute__((always_inline)) {
                    LOAD_STAGE_SLOT(slot, w1);
                    up_init(ch, accA);
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int ntl = 0; ntl < 2; ++ntl) accA[ntl][0] = DT::mfma32(w1[ntl * KC + c], hf[0][c].v, accA[ntl][0]);
                };
                auto down = [&](int slot) __attribute__((always_inline)) {
                    LOAD_STAGE_SLOT(slot, w2);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) x[0][nt] = DT::mfma32(w2[nt], hidA[0].v, x[0][nt]);
                };
                auto activate = [&]() __attribute__((always_inline)) { act4(accA[0][0], hidA[0], 0); act4(accA[1][0], hidA[0], 1); };
                ADV(4); up(0, 0);
                for (int ch2 = 0; ch2 < nch - 2; ch2 += 2) {
                    activate();                              // chunk ch2
                    ADV(5); up(ch2 + 1, 1);
                    ADV(6); down(0);
                    activate();                              // chunk ch2 + 1
                    ADV(7); up(ch2 + 2, 1);
                    ADV(8); down(0);
                }
                activate();                                  // chunk nch - 2
                ADV(5); up(nch - 1, 1);
                ADV(6); down(0);
                activate();                                  // chunk nch - 1
                ADV(7); down(1);                             // stage 3 + 2 nch
            } else {
                {   // prologue: up-projection of chunk 0, activation of its lower row tiles
                    ADVANCE(0);
                    LOAD_STAGE(0, w1);
                    up_init(0, accA);
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                            for (int rt = 0; rt < RT; ++rt) accA[ntl][rt] = DT::mfma32(w1[ntl * KC + c], hf[rt][c].v, accA[ntl][rt]);
#pragma unroll
                    for (int rt = 0; rt < RH; ++rt) { act4(accA[0][rt], hidA[rt], 0); act4(accA[1][rt], hidA[rt], 1); }
                }
                for (int ch = 0; ch < nch - 1; ++ch) {
                    f32x4 accB[2][RT];
                    Frag8 hidB[RT];
                    float ga[RH > 0 ? RH : 1][8];       // activations of the half in flight, fp32 until packed
                    {   // phase 1
                        ADVANCE(1);
                        LOAD_STAGE(1, w1);
                        up_init(ch + 1, accB);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int c = 0; c < KC; ++c)
#pragma unroll
                            for (int ntl = 0; ntl < 2; ++ntl) {
                                // slice sl = (c, ntl): one hidden unit per upper row tile, element (sl >> 2, sl & 3).
                                // Issue order MFMA, 2 VALU, MFMA, rest: a 16-cycle MFMA lets two VALU ops issue under it,
                                // and back-to-back MFMAs would leave the first one's slots empty (in-order issue).
                                const int sl = c * 2 + ntl;                    // 0..7
                                Act16Head hd[RH > 0 ? RH : 1];
#pragma unroll
                                for (int rt = 0; rt < RT; ++rt) {
                                    accB[ntl][rt] = DT::mfma32(w1[ntl * KC + c], hf[rt][c].v, accB[ntl][rt]);
                                    __builtin_amdgcn_sched_barrier(0);
                                    if (rt == 0) {
#pragma unroll
                                        for (int r2 = 0; r2 < RH; ++r2) hd[r2] = act16_head<ACT>(accA[sl >> 2][RH + r2][sl & 3]);
                                        __builtin_amdgcn_sched_barrier(0);
                                    }
                                }
#pragma unroll
                                for (int rt = 0; rt < RH; ++rt) ga[rt][sl] = act16_tail<ACT>(accA[sl >> 2][RH + rt][sl & 3], hd[rt]);
                                __builtin_amdgcn_sched_barrier(0);
                            }
#pragma unroll
                        for (int rt = 0; rt < RH; ++rt)
#pragma unroll
                            for (int w = 0; w < 4; ++w) hidA[RH + rt].w[w] = pack2<DT>(ga[rt][2 * w], ga[rt][2 * w + 1]);
                    }
                    {   // phase 2
                        ADVANCE(0);
                        LOAD_STAGE(0, w2);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) {
                            Act16Head hd[RH > 0 ? RH : 1];
#pragma unroll
                            for (int rt = 0; rt < RT; ++rt) {
                                x[rt][nt] = DT::mfma32(w2[nt], hidA[rt].v, x[rt][nt]);
                                __builtin_amdgcn_sched_barrier(0);
                                if (rt == 0) {
#pragma unroll
                                    for (int r2 = 0; r2 < RH; ++r2) hd[r2] = act16_head<ACT>(accB[nt >> 2][r2][nt & 3]);
                                    __builtin_amdgcn_sched_barrier(0);
                                }
                            }
#pragma unroll
                            for (int rt = 0; rt < RH; ++rt) ga[rt][nt] = act16_tail<ACT>(accB[nt >> 2][rt][nt & 3], hd[rt]);
                            __builtin_amdgcn_sched_barrier(0);
                        }
#pragma unroll
                        for (int rt = 0; rt < RH; ++rt)
#pragma unroll
                            for (int w = 0; w < 4; ++w) hidB[rt].w[w] = pack2<DT>(ga[rt][2 * w], ga[rt][2 * w + 1]);
                    }
#pragma unroll
                    for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt) accA[ntl][rt] = accB[ntl][rt];
#pragma unroll
                    for (int rt = 0; rt < RH; ++rt) hidA[rt] = hidB[rt];
                }
                {   // epilogue: last chunk's upper-half activation, then its down-projection
#pragma unroll
                    for (int rt = RH; rt < RT; ++rt) { act4(accA[0][rt], hidA[rt], 0); act4(accA[1][rt], hidA[rt], 1); }
                    ADVANCE(1);
                    LOAD_STAGE(1, w2);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt) x[rt][nt] = DT::mfma32(w2[nt], hidA[rt].v, x[rt][nt]);
                }
            }
        };

        // ---- 29*K + 1 output projection (8 stages); rf[i] = operand fragments whose rows are envs,
        //      row r16 being env lane_env (stored when lane_ok) ----
        auto heads = [&](auto& rf, const int64_t lane_env, const bool lane_ok, const float* fvp) __attribute__((always_inline)) {
            constexpr int NR = sizeof(rf) / sizeof(rf[0]);
            static_assert(NR == 1, "one operand tile per wave: row r16 is the env lane_env");
            // The outputs stay in registers until the last stage has been consumed: stores count in the same
            // in-order vmcnt queue as the weight prefetches, so a store issued inside the stage loop would make
            // the next stage's wait sit out an HBM write.
            f32x4 res[HEAD_TILES][NR];
#pragma unroll
            for (int st = 0; st < HEAD_STAGES; ++st) {
                ADV(st);                    // a multiple of 4 stages precedes the readout in the TAIL launch, an even number otherwise
                LOAD_STAGE(st & 1, wf);
#pragma unroll
                for (int ntl = 0; ntl < 2; ++ntl) {
                    const int nt = 2 * st + ntl;
                    const float4 b = *reinterpret_cast<const float4*>(fvp + FV_BH + 16 * nt + 4 * g);
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        f32x4 acc = {b.x, b.y, b.z, b.w};
#pragma unroll
                        for (int c = 0; c < KC; ++c) acc = DT::mfma32(wf[ntl * KC + c], rf[i][c].v, acc);
                        res[nt][i] = acc;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int64_t env = lane_env;
                if (lane_ok) {
                    // a lane holds 4 consecutive outputs of its row: one 4-dword store (rows are only dword-aligned:
                    // the type says so and the compiler picks the widest store the target allows at that alignment)
                    typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
                    float* lrow = a.logits + env * a.n_logits;
#pragma unroll
                    for (int nt = 0; nt < HEAD_TILES; ++nt) {
                        const int col0 = 16 * nt + 4 * g;
                        if (col0 + 3 < a.n_logits) {
                            *reinterpret_cast<f32x4_a4*>(lrow + col0) = (f32x4_a4){res[nt][i][0], res[nt][i][1], res[nt][i][2], res[nt][i][3]};
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int col = col0 + e;
                                if (col < a.n_logits) lrow[col] = res[nt][i][e];
                                else if (col == a.n_logits) a.value[env] = res[nt][i][e];
                            }
                        }
                    }
                }
            }
        };
        const float* fv = vlds + V_LAYER0 + a.n_layers * lv_size(a.F);

        if constexpr (!TAILP) {
            // ================= tokenizer: K = [obj 16 | prop <= 112], N = d =================
            Frag8 e[RT][KC];
            // PACK: the env of this lane's row r16 and the row's token index inside it (otherwise a tile is one env and
            // both follow from the tile index: nothing is kept in registers)
            int64_t lenv[PACK ? RT : 1];
            int ltok[PACK ? RT : 1];
            auto env_at = [&](int rt) __attribute__((always_inline)) -> int64_t {
                if (PACK) return lenv[PACK ? rt : 0];
                const int64_t env = env0 + rt;
                return env < a.B ? env : a.B - 1;
            };
            auto tok_at = [&](int rt) __attribute__((always_inline)) { return PACK ? ltok[PACK ? rt : 0] : r16; };
            int n_park = 0;             // MERGE: token-0 rows this wave parks in this pass (wave-uniform)
            int now_pr[PACK ? KRT : 1][4];
            if (INK && !(RT == KRT && have_pre)) ink_entries(__builtin_amdgcn_readfirstlane((int)env0), now_pr);   // no entries from the pass before: select them now
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (PACK) {
                    int e0, e1, e2, e3;
                    if (RT == KRT && have_pre) {
                        e0 = pre_pr[PACK ? rt : 0][0]; e1 = pre_pr[PACK ? rt : 0][1]; e2 = pre_pr[PACK ? rt : 0][2]; e3 = pre_pr[PACK ? rt : 0][3];
                    } else if (INK) {
                        e0 = now_pr[PACK ? rt : 0][0]; e1 = now_pr[PACK ? rt : 0][1]; e2 = now_pr[PACK ? rt : 0][2]; e3 = now_pr[PACK ? rt : 0][3];
                    } else {
                        int64_t tix = env0 + rt; tix = tix < n_units ? tix : n_units - 1;
                        const int4 pr = a.pairs[tix];
                        e0 = __builtin_amdgcn_readfirstlane(pr.x); e1 = __builtin_amdgcn_readfirstlane(pr.y);
                        e2 = __builtin_amdgcn_readfirstlane(pr.z); e3 = __builtin_amdgcn_readfirstlane(pr.w);
                    }
                    // the slot (rows 4 s .. 4 s + 3) an env starts in, for this lane's row and for its 4 keys (one slot)
                    auto owner = [&](int sl) __attribute__((always_inline)) {
                        int o = 0;
                        o = (sl >= 1 && e1 >= 0) ? 1 : o;
                        o = (sl >= 2 && e2 >= 0) ? 2 : o;
                        o = (sl >= 3 && e3 >= 0) ? 3 : o;
                        return o;
                    };
                    if (env0 + rt < n_units) n_park += 1 + (e1 >= 0 ? 1 : 0) + (e2 >= 0 ? 1 : 0) + (e3 >= 0 ? 1 : 0);
                    const int orow = owner(r16 >> 2), okey = owner(g);
                    const int64_t le = orow == 0 ? e0 : orow == 1 ? e1 : orow == 2 ? e2 : e3;
                    lenv[PACK ? rt : 0] = le;
                    ltok[PACK ? rt : 0] = r16 - 4 * orow;
                    const int nvalid = a.n_valid[le];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        kmask[rt][i] = (okey == orow && 4 * g + i - 4 * okey <= nvalid) ? 0.f : -INFINITY;
                } else {
                    const int64_t env = env_at(rt);
                    const int nvalid = a.n_valid ? a.n_valid[env] : T - 1;
#pragma unroll
                    for (int i = 0; i < 4; ++i) kmask[rt][i] = (4 * g + i) <= nvalid ? 0.f : -INFINITY;
                    if (env0 + rt < a.B) n_park += 1;
                }
            }
            // MERGE: reserve this wave's entries of the workgroup's tail list now, so that the count of waiting envs is
            // known to every wave behind the pass's first barrier (merge_decide), long before the stage fetch reaches
            // the end of this segment
            int t_pos = 0;
            if (MERGE) {
                if (lane == 0) t_pos = __hip_atomic_fetch_add(&tail_wr, n_park, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                t_pos = __builtin_amdgcn_readfirstlane(t_pos);
            }
            int4 nxt[PACK ? RT : 1];
            if (PACK && !INK && RT == KRT && next_wg0 >= 0) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    int64_t tix = next_wg0 + (int64_t)wave * KRT + rt; tix = tix < n_units ? tix : n_units - 1;
                    nxt[PACK ? rt : 0] = a.pairs[tix];
                }
            }
            if (a.tok_vec) {
                // a lane's 8 k slots per chunk are two runs of 4 consecutive obs lanes: k0 = 32 c + 4 g + 16 jh.
                // Only (c, jh) = (0, 0) falls in the object block (rows 1..15); every other run is proprio (row 0).
                // The lane coordinates go through an opaque copy: the 16 slot offsets and masks derived from them are
                // tile-invariant, and hoisted out of the tile loop they would sit in (spilled) registers for the whole tile.
                int tr = r16, tg = g;
                asm volatile("" : "+v"(tr), "+v"(tg));
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const float* orow = static_cast<const float*>(a.obs) + env_at(rt) * a.obs_ld;
                    const int tk = PACK ? tok_at(rt) : tr;                         // the row's token index
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int jh = 0; jh < 2; ++jh) {
                            const int k0 = 32 * c + 4 * tg + 16 * jh;
                            bool valid; int idx;
                            if (c == 0 && jh == 0) { valid = tk >= 1; idx = a.prop_dim + (tk - 1) * 16 + k0; }
                            else { valid = tk == 0 && (k0 - 16) < a.prop_dim; idx = k0 - 16; }
                            const float4 v = *reinterpret_cast<const float4*>(orow + (valid ? idx : 0));
                            const uint32_t lo = pack2<DT>(v.x, v.y), hi = pack2<DT>(v.z, v.w);
                            e[rt][c].w[2 * jh] = valid ? lo : 0u;
                            e[rt][c].w[2 * jh + 1] = valid ? hi : 0u;
                        }
                }
            } else {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const int64_t env = env_at(rt);
                    const int tk = tok_at(rt);
                    float ev[KC][8];
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const int k = 32 * c + 4 * g + (j & 3) + (j >> 2) * 16;    // permuted k order
                            int idx; bool on;
                            if (k < 16) { on = tk >= 1 && k < a.obj_dim; idx = a.prop_dim + (tk - 1) * a.obj_dim + k; }
                            else { on = tk == 0 && (k - 16) < a.prop_dim; idx = k - 16; }
                            float v = 0.f;
                            if (on) {
                                const int64_t off = env * a.obs_ld + idx;
                                v = a.obs_f32 ? static_cast<const float*>(a.obs)[off] : DT::to_f(static_cast<const u16*>(a.obs)[off]);
                            }
                            ev[c][j] = v;
                        }
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int w = 0; w < 4; ++w) e[rt][c].w[w] = pack2<DT>(ev[c][2 * w], ev[c][2 * w + 1]);
                }
            }
            // RING: the tile's own loads (obs, key counts) are waited for HERE, with the wait the compiler can see
            // (vmcnt(0); expcnt / lgkmcnt left at their maxima).  It does not know of the ring's loads, so wherever it
            // later met a value of its own still in flight - or reused such a register - it would wait for "all
            // outstanding loads", i.e. drain the ring in mid-tile; after this it has nothing pending.
            // INK: the next pass's entries are selected HERE, between this pass's input loads and their wait
            if (INK && RT == KRT) {
                have_pre = next_wg0 >= 0;
                if (have_pre) ink_entries((int)next_wg0 + uwave * KRT, pre_pr);
            }
            if (RING || DMA) __builtin_amdgcn_s_waitcnt(0x0F70);
            if (PACK && !INK && RT == KRT) {
                have_pre = next_wg0 >= 0;
                if (have_pre) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        pre_pr[PACK ? rt : 0][0] = __builtin_amdgcn_readfirstlane(nxt[PACK ? rt : 0].x);
                        pre_pr[PACK ? rt : 0][1] = __builtin_amdgcn_readfirstlane(nxt[PACK ? rt : 0].y);
                        pre_pr[PACK ? rt : 0][2] = __builtin_amdgcn_readfirstlane(nxt[PACK ? rt : 0].z);
                        pre_pr[PACK ? rt : 0][3] = __builtin_amdgcn_readfirstlane(nxt[PACK ? rt : 0].w);
                    }
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float4 bp = *reinterpret_cast<const float4*>(vlds + V_BP + 16 * nt + 4 * g);
                const float4 bo = *reinterpret_cast<const float4*>(vlds + V_BO + 16 * nt + 4 * g);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const float4 b = tok_at(rt) == 0 ? bp : bo;
                    x[rt][nt] = (f32x4){b.x, b.y, b.z, b.w};
                }
            }
#pragma unroll
            for (int st = 0; st < EMB_STAGES; ++st) {
                ADVANCE(st & 1);
                if (st == 0) merge_decide();
                LOAD_STAGE(st & 1, wf);
#pragma unroll
                for (int c = 0; c < KC; ++c)
#pragma unroll
                    for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt) x[rt][2 * st + ntl] = DT::mfma32(wf[ntl * KC + c], e[rt][c].v, x[rt][2 * st + ntl]);
            }
            // ================= transformer blocks =================
            const int dense_layers = MODE == MODE_FULL ? a.n_layers : a.n_layers - 1;
            for (int l = 0; l < dense_layers; ++l) {
                const float* lv = vlds + V_LAYER0 + l * lv_size(a.F);
                attention(lv);
                proj_and_ffn(lv);
            }
            if (MODE == MODE_HEAD) {
                // last block: attention only, then park token 0 (lanes r16 == 0) for the TAIL launch
                attention(vlds + V_LAYER0 + (a.n_layers - 1) * lv_size(a.F));
                if (MERGE) {
                    // the parked envs' ids -> the entries reserved at the start of the pass (lanes 0..15 speak for their
                    // row; an env's place among the wave's entries is its rank among the parking lanes)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        const int64_t env = PACK ? lenv[PACK ? rt : 0] : env0 + rt;
                        const bool parks = (PACK ? ((r16 & 3) == 0 && ltok[PACK ? rt : 0] == 0 && env0 + rt < n_units)
                                                 : (r16 == 0 && env < a.B)) && g == 0;
                        const uint64_t who = __ballot(parks);
                        if (parks) tail_list[(t_pos + __popcll(who & ((1ull << lane) - 1))) & (TAIL_CAP - 1)] = (int)env;
                        t_pos += __popcll(who);
                    }
                }
                if (PACK ? (r16 & 3) == 0 : r16 == 0) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        // PACK: the first row of every occupied slot is token 0 of an env; units past the end are
                        // recomputed copies of the last tile and store nothing
                        const int64_t env = PACK ? lenv[PACK ? rt : 0] : env0 + rt;
                        if (PACK ? (ltok[PACK ? rt : 0] == 0 && env0 + rt < n_units) : env < a.B) {
                            uint4* dst = reinterpret_cast<uint4*>(a.ws + (env * 4 + g) * WS_DWORDS);
#pragma unroll
                            for (int nt = 0; nt < NT; ++nt) dst[nt] = __builtin_bit_cast(uint4, x[rt][nt]);
#pragma unroll
                            for (int c = 0; c < KC; ++c) dst[NT + c] = of[rt][c].u;
                        }
                    }
                }
                // MERGE: the lanes rejoin HERE, in a block of their own.  Without it the join of the lane-dependent
                // branches above is the head of the tail-pass loop that follows the pass, and the compiler's uniformity
                // analysis then takes every value that loop carries - the stage-fetch offsets among them, which must
                // be scalar operands of the transfer instructions - for lane-dependent.
                if (MERGE) asm volatile("" ::: "memory");
            } else {
                // ================= readout: token 0 of every env -> 29*K logits + value =================
                Frag8 yf[RT][KC];
                norm_to_frags(fv + FV_LNG, fv + FV_LNB, a.final_ln != 0, yf);
                Frag8 rf[1][KC];        // B operand: lane (env r16 < RT, group g)
#pragma unroll
                for (int c = 0; c < KC; ++c) rf[0][c].u = make_uint4(0, 0, 0, 0);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int c = 0; c < KC; ++c)
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            // row 0 of this env's tile sits in lanes 16*g; hand it to lane (r16 == rt, g)
                            const uint32_t v = __shfl(yf[rt][c].w[w], 16 * g, WAVE);
                            if (r16 == rt) rf[0][c].w[w] = v;
                        }
                heads(rf, env0 + r16, r16 < RT && env0 + r16 < a.B, fv);
            }
        } else {
            // ================= TAIL: rows are envs (token 0 of each) =================
            const float* lv = vlds + V_LAYER0 + (a.n_layers - 1) * lv_size(a.F);
            int64_t tenv = env0 + r16;                     // this lane's row
            bool tok = tenv < a.B;
            if (decltype(tail_tag)::value) {
                // MERGE: the next (at most) 64 envs of the workgroup's list, 16 to a wave.  Their rows were parked by
                // this workgroup's own waves: once every wave's stores have completed (vmcnt) and every wave has said
                // so (barrier), the rows and the list entries are readable - the waves of a workgroup share the CU's
                // vector cache, and nothing else ever read these lines in this launch.
                const int n = t_cnt < TAIL_WG_ENVS ? t_cnt : TAIL_WG_ENVS, base = t_rd;
                t_rd += n; t_cnt -= n;
                t_tail_next = !t_more_head && t_cnt > 0;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                lds_barrier();
                const int idx = wave * TAIL_ENVS + r16;
                tok = idx < n;                             // rows past the list's end compute on the first env's row and store nothing
                tenv = tail_list[(base + (tok ? idx : 0)) & (TAIL_CAP - 1)];
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                int64_t env = decltype(tail_tag)::value ? tenv : env0 + rt * TAIL_ENVS + r16;
                env = env < a.B ? env : a.B - 1;           // rows >= TAIL_ENVS: never stored
#pragma unroll
                for (int i = 0; i < 4; ++i) kmask[rt][i] = 0.f;
                const uint4* src = reinterpret_cast<const uint4*>(a.ws + (env * 4 + g) * WS_DWORDS);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) x[rt][nt] = __builtin_bit_cast(f32x4, src[nt]);
#pragma unroll
                for (int c = 0; c < KC; ++c) of[rt][c].u = src[NT + c];
            }
            // MERGE: the rows are waited for here, with the wait the compiler can see (as the tokenizer's loads are)
            if (decltype(tail_tag)::value) __builtin_amdgcn_s_waitcnt(0x0F70);
            proj_and_ffn(lv);
            Frag8 yf[RT][KC];
            norm_to_frags(fv + FV_LNG, fv + FV_LNB, a.final_ln != 0, yf);
            heads(yf, tenv, tok, fv);
        }
    };
    typedef std::integral_constant<int, KRT> rt_bulk;

    // PACK: the remainder of the last round runs as ONE-tile passes.  A SIMD turns out tiles at a fixed rate whether it
    // holds one wave or two, so what counts is tiles per SIMD; workgroups b and b + CUs share a CU.  With P two-tile
    // workgroup passes, the r = P mod CUs passes past the last multiple of the CU count put a second (or third) pass on r
    // CUs: those few tiles then cost a whole two-tile pass time at the end of the launch (the headline batch: 1283 passes,
    // r = 3: 23 tiles = the last 24 us of 143).  When r is small, the tiles of those r passes go instead, four to a
    // workgroup and one to a wave, to the workgroups that idle in that round: half the added time, on twice the CUs.
    int64_t n_bulk = ntiles;                 // workgroup passes of the bulk body
    int64_t rem_tile0 = 0; int rem_first_wg = 0, rem_passes = 0;
    if (PACK && KRT == 2 && a.cus > 0) {
        // (32-bit arithmetic: the packed tile count is an int32, and a 64-bit division is a ~200-instruction routine
        // of which three sat between the prologue and the first pass)
        const uint32_t nt32 = (uint32_t)ntiles;
        const int64_t r = nt32 % (uint32_t)a.cus;
        const int64_t p2 = nt32 - (uint32_t)r;
        const int64_t nrem = n_units - p2 * ENVS_PER_WG;                 // tiles left for one-tile passes
        const int q = (int)(((uint32_t)nrem + 3u) / 4u), fb = (int)((uint32_t)p2 % gridDim.x);
        if (r > 0 && r <= 32 && p2 > 0 && fb + q <= (int)gridDim.x) { n_bulk = p2; rem_tile0 = p2 * ENVS_PER_WG; rem_first_wg = fb; rem_passes = q; }
    }
    typedef std::integral_constant<int, 1> rt_one;
    typedef std::false_type head_pass;
    if constexpr (MERGE) {
        // head-type passes (this workgroup's one-tile remainder pass first, if it has one, then its bulk passes), each
        // followed by the tail passes it has made due: one whenever 64 envs wait, and the rest after the last head-type
        // pass.  The remainder pass goes FIRST: the workgroups that get one are the younger of their CU's two, and a
        // pass is a latency chain of 64 stages - run while the CU's other workgroup computes it costs the CU its
        // arithmetic (half a bulk pass); run at the end, after that workgroup has left, it cost the whole chain
        // (~18 us at the end of the launch, on 6 CUs of 256, at the headline batch).
        const int qi = (int)blockIdx.x - rem_first_wg;
        bool rem_due = PACK && KRT == 2 && qi >= 0 && qi < rem_passes;
        int64_t tile = blockIdx.x;
        while (true) {
            if (rem_due) {
                rem_due = false;
                t_more_head = tile < n_bulk;
                // ... and at raised priority: this workgroup's chain of passes is one longer than every other's, so
                // while it runs the extra one it goes first at the SIMDs' issue ports
                __builtin_amdgcn_s_setprio(3);
                pass(rt_one(), head_pass(), rem_tile0 + (int64_t)qi * 4 + uwave, -1);
                __builtin_amdgcn_s_setprio(0);
            } else if (tile < n_bulk) {
                const int64_t env0 = tile * ENVS_PER_WG + (int64_t)uwave * KRT * ENVS_PER_TILE;
                const int64_t ntile = tile + gridDim.x;
                t_more_head = ntile < n_bulk;
                pass(rt_bulk(), head_pass(), env0, (PACK && ntile < n_bulk) ? ntile * ENVS_PER_WG : -1);
                tile = ntile;
            } else break;
            while (t_tail_next) pass(rt_one(), std::integral_constant<bool, MERGE>(), 0, -1);
        }
    } else {
        for (int64_t tile = blockIdx.x; tile < n_bulk; tile += gridDim.x) {
            const int64_t env0 = RING ? tile * a.ring_epw + uwave : tile * ENVS_PER_WG + (int64_t)wave * KRT * ENVS_PER_TILE;
            if (RING && (uwave >= a.ring_epw || env0 >= a.B)) {
                // a wave without an env: it keeps its share of the weight ring moving (loads, waits, barriers - exactly one
                // advance per stage, like the working waves) and reads no fragment, so the workgroup's LDS reads are those
                // of its working waves only
                for (int s_ = a.s_begin; s_ < a.s_end; ++s_) ring_advance();
                continue;
            }
            const int64_t ntile = tile + gridDim.x;
            pass(rt_bulk(), head_pass(), env0, (PACK && ntile < n_bulk) ? ntile * ENVS_PER_WG : -1);
        }
        if (PACK && KRT == 2) {
            const int qi = (int)blockIdx.x - rem_first_wg;
            if (qi >= 0 && qi < rem_passes) pass(rt_one(), head_pass(), rem_tile0 + (int64_t)qi * 4 + wave, -1);
        }
    }
    if (RING || DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // no transfer into LDS may outlive the workgroup
    lds_barrier();   // every wave leaves together; no LDS slot is read after this point
}

// ---- weight image ------------------------------------------------------------------
struct PackArgs {
    bsrl_cfg_params p;
    void* frags; float* vec;
    int n_layers, F, n_stages, n_out, prop_dim, obj_dim, final_ln;
};

__device__ __forceinline__ int perm_k(int c, int gg, int j) { return 32 * c + 4 * gg + (j & 3) + (j >> 2) * 16; }

// one wave per fragment, one lane per 16-byte slot
template <typename DT>
__global__ __launch_bounds__(256) void cfg_pack_frags_kernel(PackArgs a) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= a.n_stages * STAGE_FRAGS) return;
    const int n16 = lane & 15, gg = lane >> 4;
    const int lstages = layer_stages(a.F);
    const int emb_end = EMB_STAGES * STAGE_FRAGS;
    const int layers_end = emb_end + a.n_layers * lstages * STAGE_FRAGS;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = 0.f;
    if (f < emb_end) {
        const int st = f / 8, r = f % 8, nt = 2 * st + r / KC, c = r % KC, n = 16 * nt + n16;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = perm_k(c, gg, j);
            if (k < 16) { if (k < a.obj_dim) v[j] = a.p.obj_w[n * a.obj_dim + k]; }
            else if (k - 16 < a.prop_dim) v[j] = a.p.prop_w[n * a.prop_dim + (k - 16)];
        }
    } else if (f < layers_end) {
        const int l = (f - emb_end) / (lstages * 8), r = (f - emb_end) % (lstages * 8);
        const float* src; int ld, n, kbase = 0, c;
        if (r < 3 * H * 8) {
            const int hd = r / 24, rr = r % 24, part = rr / 8, q = rr % 8;
            src = part == 0 ? a.p.blk[l].q_w : part == 1 ? a.p.blk[l].k_w : a.p.blk[l].v_w;
            ld = D; n = 32 * hd + 16 * (q / KC) + n16; c = q % KC;
        } else if (r < 3 * H * 8 + NT * KC) {
            const int r2 = r - 3 * H * 8;
            src = a.p.blk[l].out_w; ld = D; n = 16 * (r2 / KC) + n16; c = r2 % KC;
        } else {
            // FFN stage order: W1(0), {W1(ch+1), W2(ch)} for ch = 0..nch-2, W2(nch-1)
            const int r3 = r - 3 * H * 8 - NT * KC, s3 = r3 / 8, q = r3 % 8, nch = a.F / 32;
            bool up; int ch;
            if (s3 == 0) { up = true; ch = 0; }
            else if (s3 == 2 * nch - 1) { up = false; ch = nch - 1; }
            else { up = ((s3 - 1) & 1) == 0; ch = (s3 - 1) / 2 + (up ? 1 : 0); }
            if (up) { src = a.p.blk[l].ffn0_w; ld = D; n = 32 * ch + 16 * (q / KC) + n16; c = q % KC; }
            else { src = a.p.blk[l].ffn2_w; ld = a.F; n = 16 * q + n16; c = 0; kbase = 32 * ch; }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = src[(int64_t)n * ld + kbase + perm_k(c, gg, j)];
    } else {
        const int r = f - layers_end, n = 16 * (r / KC) + n16, c = r % KC;
        if (n < a.n_out) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = a.p.heads_w[n * D + perm_k(c, gg, j)];
        }
    }
    uint4 o;
    o.x = pack2<DT>(v[0], v[1]); o.y = pack2<DT>(v[2], v[3]); o.z = pack2<DT>(v[4], v[5]); o.w = pack2<DT>(v[6], v[7]);
    static_cast<uint4*>(a.frags)[(int64_t)f * 64 + lane] = o;
}

__global__ __launch_bounds__(256) void cfg_pack_vec_kernel(PackArgs a) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int total = vec_floats(a.n_layers, a.F);
    if (i >= total) return;
    float v = 0.f;
    if (i < V_LAYER0) v = i < V_BO ? a.p.prop_b[i] : a.p.obj_b[i - V_BO];
    else if (i < V_LAYER0 + a.n_layers * lv_size(a.F)) {
        const int l = (i - V_LAYER0) / lv_size(a.F), r = (i - V_LAYER0) % lv_size(a.F);
        const auto& b = a.p.blk[l];
        if (r < LV_B1) {
            const float* srcs[8] = {b.ln_attn_w, b.ln_attn_b, b.q_b, b.k_b, b.v_b, b.out_b, b.ln_ffn_w, b.ln_ffn_b};
            v = srcs[r / D][r % D];
        } else if (r < lv_b2(a.F)) v = b.ffn0_b[r - LV_B1];
        else v = b.ffn2_b[r - lv_b2(a.F)];
    } else {
        const int r = i - V_LAYER0 - a.n_layers * lv_size(a.F);
        if (r < FV_LNB) v = a.final_ln ? a.p.final_ln_w[r] : 1.f;
        else if (r < FV_BH) v = a.final_ln ? a.p.final_ln_b[r - FV_LNB] : 0.f;
        else v = (r - FV_BH) < a.n_out ? a.p.heads_b[r - FV_BH] : 0.f;
    }
    a.vec[i] = v;
}

bool shape_ok(const bsrl_cfg_desc* d) {
    return d && d->d == D && d->n_heads == H && d->T == T && d->ffn > 0 && d->ffn % 32 == 0 && d->ffn <= 4096 &&
           d->n_layers >= 1 && d->n_layers <= BSRL_MAX_LAYERS && (d->dtype == BSRL_F16 || d->dtype == BSRL_BF16) &&
           d->obj_dim >= 1 && d->obj_dim <= 16 && d->prop_dim >= 1 && d->prop_dim <= D - 16 &&
           d->n_gears >= 1 && 29 * d->n_gears + 1 <= HEAD_TILES * 16 && (d->act == BSRL_ACT_GELU || d->act == BSRL_ACT_RELU);
}
int64_t frag_bytes(const bsrl_cfg_desc* d) { return (int64_t)total_stages(d->n_layers, d->ffn) * STAGE_U4 * 16; }

// Tile table of the packed HEAD launch.  Classes by token count (1 + n_valid): tiny <= 4, mid 5..8, host 9..12, long
// the rest; each class keeps env order (a stable split, so the table is a function of the batch alone).  Tiles, in
// this order: the mid pairs (mid[2 i], mid[2 i + 1]) at rows 0 / 8 (a lone last one if their count is odd); the quads
// of the tiny envs that found no host, at rows 0 / 4 / 8 / 12 (the last tile may hold fewer); one tile per host env,
// host[i] at rows 0..11 with tiny[i] at rows 12..15 while tiny envs last; one tile per long env.
// pairs[t] = the env that starts in each 4-row slot, -1 where the slot continues the env before it (or is empty);
// *n_packed = the number of tiles.
// Workgroup b owns the envs [b span, (b + 1) span), `per` consecutive ones per thread.  Every workgroup counts the
// classes of the WHOLE batch for itself (coalesced 16-byte reads out of L2: cheaper than a second launch or a
// cross-workgroup hand-off), which gives it both the counts before its span and the totals.
constexpr int PAIR_THREADS = 256;
constexpr int PAIR_MAX_WGS = 256;
constexpr int PAIR_OWN = 4;                                // own envs a thread keeps in registers
constexpr int PAIR_CNT = 16;                               // 16-byte loads (4 key counts each) per thread and counting pass
__device__ __forceinline__ int env_tiny(int nv) { return nv >= 0 && nv <= 3 ? 1 : 0; }
__device__ __forceinline__ int env_mid(int nv) { return nv >= 4 && nv <= 7 ? 1 : 0; }
__device__ __forceinline__ int env_host(int nv) { return nv >= 8 && nv <= 11 ? 1 : 0; }
__global__ __launch_bounds__(PAIR_THREADS) void cfg_pair_kernel(const int32_t* n_valid, int64_t B, int64_t span, int per,
                                                                int4* pairs, int32_t* n_packed) {
    __shared__ int red[9][PAIR_THREADS / WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t w0 = (int64_t)blockIdx.x * span;
    // Every global load of the common case leaves in one batch (own envs first, then PAIR_CNT loads per thread per
    // pass): a dependent round trip costs ~1.5 us on an otherwise idle chip, and this kernel is nothing but round trips.
    const int64_t lo = w0 + (int64_t)tid * per < B ? w0 + (int64_t)tid * per : B;
    const int64_t hi = lo + per < B ? lo + per : B;
    int own[PAIR_OWN];
#pragma unroll
    for (int j = 0; j < PAIR_OWN; ++j) {       // clamped index, not a guarded load: a load under a branch is waited for at once
        const int v = n_valid[lo + j < B ? lo + j : B - 1];
        own[j] = lo + j < hi ? v : -1;
    }
    // class counts of the whole batch, four envs per load (n_valid is 16-byte aligned on this path, B < 2^31):
    // [0] tiny, [1] mid, [2] host; b* = before this workgroup's span, t* = in total
    int bt = 0, bm = 0, bh = 0, tt = 0, tm = 0, th = 0;
    const int nq = (int)(B >> 2), w0q = (int)(w0 >> 2);     // w0 is a multiple of PAIR_THREADS
    const int4* nvq = reinterpret_cast<const int4*>(n_valid);
    for (int q0 = 0; q0 < nq; q0 += PAIR_CNT * PAIR_THREADS) {
        int4 v[PAIR_CNT];
#pragma unroll
        for (int j = 0; j < PAIR_CNT; ++j) { const int q = q0 + j * PAIR_THREADS + tid; v[j] = nvq[q < nq ? q : nq - 1]; }
#pragma unroll
        for (int j = 0; j < PAIR_CNT; ++j) {
            const int q = q0 + j * PAIR_THREADS + tid;
            int c0 = env_tiny(v[j].x) + env_tiny(v[j].y) + env_tiny(v[j].z) + env_tiny(v[j].w);
            int c1 = env_mid(v[j].x) + env_mid(v[j].y) + env_mid(v[j].z) + env_mid(v[j].w);
            int c2 = env_host(v[j].x) + env_host(v[j].y) + env_host(v[j].z) + env_host(v[j].w);
            c0 = q < nq ? c0 : 0; c1 = q < nq ? c1 : 0; c2 = q < nq ? c2 : 0;
            tt += c0; tm += c1; th += c2;
            bt += q < w0q ? c0 : 0; bm += q < w0q ? c1 : 0; bh += q < w0q ? c2 : 0;
        }
    }
    if (tid < (int)(B & 3)) {                               // the last B % 4 envs
        const int64_t e = (int64_t)nq * 4 + tid;
        const int nv = n_valid[e];
        tt += env_tiny(nv); tm += env_mid(nv); th += env_host(nv);
        if (e < w0) { bt += env_tiny(nv); bm += env_mid(nv); bh += env_host(nv); }
    }
    // the inclusive scans of this thread's class counts over the workgroup
    int ct = 0, cm = 0, ch = 0;
    if (per <= PAIR_OWN) {
#pragma unroll
        for (int j = 0; j < PAIR_OWN; ++j) { ct += env_tiny(own[j]); cm += env_mid(own[j]); ch += env_host(own[j]); }
    } else {
        for (int64_t e = lo; e < hi; ++e) { const int nv = n_valid[e]; ct += env_tiny(nv); cm += env_mid(nv); ch += env_host(nv); }
    }
    int it = ct, im = cm, ih = ch;
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const int vt = __shfl_up(it, d, WAVE), vm = __shfl_up(im, d, WAVE), vh = __shfl_up(ih, d, WAVE);
        if (lane >= d) { it += vt; im += vm; ih += vh; }
    }
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        bt += __shfl_xor(bt, d, WAVE); bm += __shfl_xor(bm, d, WAVE); bh += __shfl_xor(bh, d, WAVE);
        tt += __shfl_xor(tt, d, WAVE); tm += __shfl_xor(tm, d, WAVE); th += __shfl_xor(th, d, WAVE);
    }
    if (lane == WAVE - 1) { red[0][wave] = it; red[1][wave] = im; red[2][wave] = ih; }
    if (lane == 0) {
        red[3][wave] = bt; red[4][wave] = bm; red[5][wave] = bh;
        red[6][wave] = tt; red[7][wave] = tm; red[8][wave] = th;
    }
    __syncthreads();
    int baset = 0, basem = 0, baseh = 0; bt = 0; bm = 0; bh = 0; tt = 0; tm = 0; th = 0;
#pragma unroll
    for (int w = 0; w < PAIR_THREADS / WAVE; ++w) {
        if (w < wave) { baset += red[0][w]; basem += red[1][w]; baseh += red[2][w]; }
        bt += red[3][w]; bm += red[4][w]; bh += red[5][w];
        tt += red[6][w]; tm += red[7][w]; th += red[8][w];
    }
    int64_t rt_ = (int64_t)bt + baset + it - ct;           // tiny envs before this thread's first env
    int64_t rm = (int64_t)bm + basem + im - cm;            // mid envs before it
    int64_t rh = (int64_t)bh + baseh + ih - ch;            // host envs before it
    int64_t rl = lo - rt_ - rm - rh;                       // long envs before it
    const int64_t loose = tt > th ? tt - th : 0;           // tiny envs without a host
    const int64_t first_quad = ((int64_t)tm + 1) / 2;
    const int64_t first_host = first_quad + (loose + 3) / 4;
    const int64_t first_long = first_host + th;
    // every slot of every tile is written exactly once: an env writes the slot it starts in and the -1 of the slots
    // that can only continue it; the last mid / loose tiny env also closes the rest of its tile, a host without a
    // tiny env its own last slot
    // (a macro, not a lambda: with the counters captured by reference the closure went through scratch memory, and a
    // kernel with a private segment pays for it at every dispatch)
#define PAIR_PLACE(E, NV)                                                                          \
    do {                                                                                           \
        const int64_t e_ = (E);                                                                    \
        const int nv_ = (NV);                                                                      \
        if (env_mid(nv_)) {                                                                        \
            int32_t* p = reinterpret_cast<int32_t*>(pairs + rm / 2) + 2 * (rm & 1);               \
            p[0] = (int32_t)e_; p[1] = -1;                                                         \
            if (rm == tm - 1 && !(rm & 1)) { p[2] = -1; p[3] = -1; }                               \
            ++rm;                                                                                  \
        } else if (env_tiny(nv_)) {                                                                \
            if (rt_ < th) {                                                                        \
                reinterpret_cast<int32_t*>(pairs + first_host + rt_)[3] = (int32_t)e_;            \
            } else {                                                                               \
                const int64_t q_ = rt_ - th;                                                       \
                int32_t* p = reinterpret_cast<int32_t*>(pairs + first_quad + q_ / 4);             \
                const int sl = (int)(q_ & 3);                                                      \
                p[sl] = (int32_t)e_;                                                               \
                if (rt_ == tt - 1) { if (sl < 1) p[1] = -1; if (sl < 2) p[2] = -1; if (sl < 3) p[3] = -1; } \
            }                                                                                      \
            ++rt_;                                                                                 \
        } else if (env_host(nv_)) {                                                                \
            int32_t* p = reinterpret_cast<int32_t*>(pairs + first_host + rh);                     \
            p[0] = (int32_t)e_; p[1] = -1; p[2] = -1;                                              \
            if (rh >= tt) p[3] = -1;                                                               \
            ++rh;                                                                                  \
        } else {                                                                                   \
            pairs[first_long + rl] = make_int4((int)e_, -1, -1, -1);                               \
            ++rl;                                                                                  \
        }                                                                                          \
    } while (0)
    if (per <= PAIR_OWN) {
#pragma unroll
        for (int j = 0; j < PAIR_OWN; ++j) if (lo + j < hi) PAIR_PLACE(lo + j, own[j]);
    } else {
        for (int64_t e = lo; e < hi; ++e) PAIR_PLACE(e, n_valid[e]);
    }
#undef PAIR_PLACE
    if (blockIdx.x == 0 && tid == 0) *n_packed = (int32_t)(first_long + (B - tt - tm - th));
}

constexpr size_t LDS_PER_WG = 160 * 1024;
size_t ring_dyn_bytes(int n_layers, int F) {
    return (size_t)((vec_floats(n_layers, F) / 4 + 63) & ~63) * 16 + (size_t)RING_SLOTS * STAGE_U4 * 16;
}

size_t dma_dyn_bytes(int n_layers, int F) {
    return (size_t)((vec_floats(n_layers, F) / 4 + 63) & ~63) * 16 + (size_t)DMA_SLOTS * STAGE_U4 * 16;
}
// two workgroups share a CU in the throughput forms: both rings must fit
bool dma_fits(int n_layers, int F) { return 2 * (dma_dyn_bytes(n_layers, F) + 2048) <= LDS_PER_WG; }

template <typename DT, int RT, int ACT, int MODE, bool PACK = false, bool RING = false, bool DMA = false, bool INK = false>
int launch_one(const FwdArgs& a, int cus, hipStream_t st) {
    const size_t dyn = RING ? ring_dyn_bytes(a.n_layers, a.F) : DMA ? dma_dyn_bytes(a.n_layers, a.F) + (INK ? INK_BYTES : 0)
                            : (size_t)vec_floats(a.n_layers, a.F) * sizeof(float);
    auto kern = cfg_forward_kernel<DT, RT, ACT, MODE, PACK, RING, DMA, INK>;
    if (dyn + sizeof(uint4) * 2 * STAGE_U4 > 64 * 1024) {       // beyond the default per-workgroup LDS window
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess)
            return BSRL_UNSUPPORTED;
    }
    const int64_t per_wg = RING ? a.ring_epw : 4 * RT * (MODE == MODE_TAIL ? TAIL_ENVS : 1);
    const int64_t ntiles = (a.B + per_wg - 1) / per_wg;
    const int64_t resident = (int64_t)cus * ((RT <= 2 && !RING) ? 2 : 1);
    hipLaunchKernelGGL(kern, dim3((unsigned)(ntiles < resident ? ntiles : resident)), dim3(256), dyn, st, a);
    return BSRL_OK;
}

template <typename DT, int ACT>
int launch_all(FwdArgs a, bool pruned, bool pack, bool latency, int cus, hipStream_t st) {
    const int ls = layer_stages(a.F), total = total_stages(a.n_layers, a.F);
    if (latency) {
        a.s_begin = 0; a.s_end = total;
        a.ring_epw = (int)((a.B + cus - 1) / cus);              // 1..4 (B <= 4 CUs): as few working waves per CU as the batch allows
        return launch_one<DT, 1, ACT, MODE_FULL, false, true>(a, cus, st);
    }
    const bool dma = dma_fits(a.n_layers, a.F);
    if (!pruned) {
        a.s_begin = 0; a.s_end = total;
        return dma ? launch_one<DT, 2, ACT, MODE_FULL, false, false, true>(a, cus, st) : launch_one<DT, 2, ACT, MODE_FULL>(a, cus, st);
    }
    const int split = EMB_STAGES + (a.n_layers - 1) * ls + 3 * H;
    a.s_begin = 0; a.s_end = split;
    a.t_begin = split; a.t_end = total;
    int rc;
    if (pack && dma && a.B <= INK_MAX_ENVS && 2 * (dma_dyn_bytes(a.n_layers, a.F) + INK_BYTES + 2048) <= LDS_PER_WG) {
        // the tile table lives in every workgroup's LDS: no table kernel (same grid sizing as below)
        return launch_one<DT, 2, ACT, MODE_HEAD, true, false, true, true>(a, cus, st);
    }
    if (pack) {
        // the grid is sized for the unpacked tile count (the packed one is known on the device only); workgroups past
        // the packed count leave after their prologue
        int64_t wgs = (a.B + PAIR_THREADS - 1) / PAIR_THREADS;
        if (wgs > PAIR_MAX_WGS) wgs = PAIR_MAX_WGS;
        const int per = (int)(((a.B + wgs - 1) / wgs + PAIR_THREADS - 1) / PAIR_THREADS);      // envs per thread
        const int64_t span = (int64_t)per * PAIR_THREADS;                                      // envs per workgroup
        wgs = (a.B + span - 1) / span;
        hipLaunchKernelGGL(cfg_pair_kernel, dim3((unsigned)wgs), dim3(PAIR_THREADS), 0, st, a.n_valid, a.B, span, per,
                           const_cast<int4*>(a.pairs), const_cast<int32_t*>(a.n_packed));
        rc = dma ? launch_one<DT, 2, ACT, MODE_HEAD, true, false, true>(a, cus, st) : launch_one<DT, 2, ACT, MODE_HEAD, true>(a, cus, st);
    } else {
        rc = dma ? launch_one<DT, 2, ACT, MODE_HEAD, false, false, true>(a, cus, st) : launch_one<DT, 2, ACT, MODE_HEAD>(a, cus, st);
    }
    if (rc != BSRL_OK || dma) return rc;           // on the direct-to-LDS pipeline the first launch runs the tail itself
    a.s_begin = split; a.s_end = total;
    return launch_one<DT, 1, ACT, MODE_TAIL>(a, cus, st);
}

}  // namespace

extern "C" int64_t bsrl_cfg_pack_size(const bsrl_cfg_desc* d) {
    if (!shape_ok(d)) return 0;
    return frag_bytes(d) + (int64_t)vec_floats(d->n_layers, d->ffn) * 4;
}

extern "C" int bsrl_cfg_pack(const bsrl_cfg_desc* d, const bsrl_cfg_params* p, void* packed, bsrl_stream stream) {
    if (!d || !p || !packed) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_pack: null pointer");
    if (!shape_ok(d)) return BSRL_UNSUPPORTED;
    if (!bsrl_aligned(packed, 16)) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_pack: image must be 16-byte aligned");
    if (!p->prop_w || !p->prop_b || !p->obj_w || !p->obj_b || !p->heads_w || !p->heads_b ||
        (d->final_ln && (!p->final_ln_w || !p->final_ln_b)))
        BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_pack: null parameter pointer");
    for (int l = 0; l < d->n_layers; ++l) {
        const float* const* q = reinterpret_cast<const float* const*>(&p->blk[l]);
        for (int i = 0; i < 16; ++i) if (!q[i]) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_pack: null parameter pointer in block %d", l);
    }
    PackArgs a;
    a.p = *p;
    a.frags = packed;
    a.vec = reinterpret_cast<float*>(static_cast<char*>(packed) + frag_bytes(d));
    a.n_layers = d->n_layers; a.F = d->ffn; a.n_stages = total_stages(d->n_layers, d->ffn);
    a.n_out = 29 * d->n_gears + 1; a.prop_dim = d->prop_dim; a.obj_dim = d->obj_dim; a.final_ln = d->final_ln;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned nf = (unsigned)(a.n_stages * STAGE_FRAGS);
    if (d->dtype == BSRL_F16) hipLaunchKernelGGL((cfg_pack_frags_kernel<F16>), dim3((nf + 3) / 4), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((cfg_pack_frags_kernel<BF16>), dim3((nf + 3) / 4), dim3(256), 0, st, a);
    hipLaunchKernelGGL(cfg_pack_vec_kernel, dim3((vec_floats(a.n_layers, a.F) + 255) / 256), dim3(256), 0, st, a);
    BSRL_CHECK_LAUNCH("bsrl_cfg_pack");
    return BSRL_OK;
}

namespace {
// workspace layout: token-0 rows (B x 768 B), then the packed launch's tile table (B int4) and its tile count
int64_t ws_rows_bytes(int64_t B) { return B * 4 * WS_DWORDS * (int64_t)sizeof(uint32_t); }
int64_t ws_pairs_bytes(int64_t B) { return B * (int64_t)sizeof(int4) + 16; }
}  // namespace

extern "C" int64_t bsrl_cfg_workspace_size(const bsrl_cfg_desc* d, int64_t B) {
    if (!shape_ok(d) || B <= 0) return 0;
    return ws_rows_bytes(B) + ws_pairs_bytes(B);
}

namespace {
// Shared body of the two forward entry points.  `rows` = the parked token-0 rows (768 B per env) or null (one-launch
// form); `table` = the packed launch's tile table (B int4 + 16 B for the tile count) or null (one env per tile).
int cfg_forward_impl(const char* who, const bsrl_cfg_desc* d, const void* packed, const void* obs, int64_t obs_ld,
                     int obs_dtype, const int32_t* n_valid, float* logits, float* value, int64_t B,
                     void* rows, void* table, hipStream_t st) {
    if (!d || !packed || !obs || !logits || !value) BSRL_FAIL(BSRL_EINVAL, "%s: null pointer", who);
    if (!shape_ok(d)) return BSRL_UNSUPPORTED;
    if (B < 0) BSRL_FAIL(BSRL_EINVAL, "%s: negative batch", who);
    if (obs_dtype != BSRL_F32 && obs_dtype != d->dtype) BSRL_FAIL(BSRL_EINVAL, "%s: obs must be F32 or the stream dtype", who);
    if (obs_ld < d->prop_dim + (d->T - 1) * d->obj_dim) BSRL_FAIL(BSRL_EINVAL, "%s: obs_ld smaller than an obs row", who);
    if (!bsrl_aligned(packed, 16)) BSRL_FAIL(BSRL_EINVAL, "%s: image must be 16-byte aligned", who);
    if (rows && !bsrl_aligned(rows, 16)) BSRL_FAIL(BSRL_EINVAL, "%s: workspace must be 16-byte aligned", who);
    if (B == 0) return BSRL_OK;
    FwdArgs a;
    a.frags = static_cast<const uint4*>(packed);
    a.vec = reinterpret_cast<const float*>(static_cast<const char*>(packed) + frag_bytes(d));
    a.obs = obs; a.obs_ld = obs_ld; a.obs_f32 = obs_dtype == BSRL_F32;
    a.tok_vec = a.obs_f32 && d->obj_dim == 16 && d->prop_dim % 4 == 0 && obs_ld % 4 == 0 && bsrl_aligned(obs, 16);
    a.n_valid = n_valid; a.logits = logits; a.value = value; a.B = B;
    a.n_layers = d->n_layers; a.F = d->ffn; a.s_begin = 0; a.s_end = 0; a.t_begin = 0; a.t_end = 0;
    a.n_logits = 29 * d->n_gears; a.final_ln = d->final_ln; a.prop_dim = d->prop_dim; a.obj_dim = d->obj_dim;
    a.ws = static_cast<uint32_t*>(rows);
    a.ring_epw = 4; a.cus = 0;
    // the TAIL launch's 4-deep weight pipeline counts stages modulo 4: it needs a hidden width that is a multiple of 64
    const bool pruned = rows && d->ffn % 64 == 0;
    // short envs share tiles when the caller gives key counts, there is room for the tile table and the descriptor
    // does not switch it off (n_valid 16-byte aligned: the table kernel reads it four at a time); B < 2^31 - 1 keeps
    // env ids in the table's int32
    const bool pack = pruned && table && n_valid && bsrl_aligned(n_valid, 16) && !(d->flags & BSRL_CFG_NO_PACK) &&
                      B < (int64_t)0x7fffffff;
    a.pairs = nullptr; a.n_packed = nullptr;
    if (pack) {
        a.pairs = static_cast<const int4*>(table);
        a.n_packed = reinterpret_cast<const int32_t*>(static_cast<const char*>(table) + ws_pairs_bytes(B) - 16);
    }
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    a.cus = cus;
    // the latency form (one launch, one env per wave, deep direct-to-LDS weight ring) for small batches, unless the
    // descriptor switches it off or vectors + ring exceed one workgroup's LDS; same output bits as the other forms
    // (and the batch is one pass of one workgroup per CU: past that the persistent loop would drain the ring once per
    // tile and the throughput forms win anyway)
    const bool latency = !(d->flags & BSRL_CFG_NO_LATENCY) && ring_dyn_bytes(d->n_layers, d->ffn) + 2048 <= LDS_PER_WG &&
                         total_stages(d->n_layers, d->ffn) >= RING_DEPTH && B <= 4 * (int64_t)cus;
    int rc;
    if (d->dtype == BSRL_F16)
        rc = d->act == BSRL_ACT_GELU ? launch_all<F16, BSRL_ACT_GELU>(a, pruned, pack, latency, cus, st) : launch_all<F16, BSRL_ACT_RELU>(a, pruned, pack, latency, cus, st);
    else
        rc = d->act == BSRL_ACT_GELU ? launch_all<BF16, BSRL_ACT_GELU>(a, pruned, pack, latency, cus, st) : launch_all<BF16, BSRL_ACT_RELU>(a, pruned, pack, latency, cus, st);
    if (rc != BSRL_OK) return rc;
    BSRL_CHECK_LAUNCH(who);
    return BSRL_OK;
}
}  // namespace

extern "C" int bsrl_cfg_forward(const bsrl_cfg_desc* d, const void* packed, const void* obs, int64_t obs_ld,
                                int obs_dtype, const int32_t* n_valid, float* logits, float* value, int64_t B,
                                void* workspace, int64_t workspace_bytes, bsrl_stream stream) {
    void* rows = nullptr;
    void* table = nullptr;
    if (workspace && B > 0 && workspace_bytes >= ws_rows_bytes(B)) {
        rows = workspace;
        if (workspace_bytes >= ws_rows_bytes(B) + ws_pairs_bytes(B)) table = static_cast<char*>(workspace) + ws_rows_bytes(B);
    }
    return cfg_forward_impl("bsrl_cfg_forward", d, packed, obs, obs_ld, obs_dtype, n_valid, logits, value, B, rows, table,
                            static_cast<hipStream_t>(stream));
}

// ---- the same forward for callers that cannot allocate ---------------------------------------------------------
// The parked rows and the tile table live in a file-scope device array instead of a caller workspace.  Every GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends.
namespace {
constexpr int64_t STATIC_MAX_ENVS = BSRL_CFG_STATIC_MAX_ENVS;
constexpr int64_t STATIC_ROWS_BYTES = STATIC_MAX_ENVS * 4 * WS_DWORDS * (int64_t)sizeof(uint32_t);
constexpr int64_t STATIC_TABLE_BYTES = STATIC_MAX_ENVS * (int64_t)sizeof(int4) + 16;
static __device__ __align__(256) unsigned char scratch[STATIC_ROWS_BYTES + STATIC_TABLE_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[MAX_DEVICES] = {};       // device address of `scratch` on each device, taken once per device

// `scratch` in host code is only a handle for the runtime: the array's device address on the current device comes from
// hipGetSymbolAddress, and that address is what kernels and copies get.
int scratch_on_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) BSRL_FAIL(BSRL_ELAUNCH, "bsrl_cfg_forward_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_forward_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            BSRL_FAIL(BSRL_ELAUNCH, "bsrl_cfg_forward_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return BSRL_OK;
}
}  // namespace

extern "C" int bsrl_cfg_forward_static(const bsrl_cfg_desc* d, const void* packed, const void* obs, int64_t obs_ld,
                                       int obs_dtype, const int32_t* n_valid, float* logits, float* value, int64_t B,
                                       bsrl_stream stream) {
    if (B > STATIC_MAX_ENVS)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_forward_static: B = %lld exceeds the built-in scratch (%lld envs); "
                  "use bsrl_cfg_forward with a workspace", (long long)B, (long long)STATIC_MAX_ENVS);
    if (d && shape_ok(d) && d->ffn % 64 != 0) return BSRL_UNSUPPORTED;    // the two-launch form needs it (see above)
    void* base = nullptr;
    const int rc = scratch_on_current_device(&base);
    if (rc != BSRL_OK) return rc;
    // fixed split of the array, whatever B: rows first, table behind the rows of the largest batch.  Nothing in either
    // part has to start at zero: the first launch writes the row of every env and every table slot the second reads.
    return cfg_forward_impl("bsrl_cfg_forward_static", d, packed, obs, obs_ld, obs_dtype, n_valid, logits, value, B,
                            base, static_cast<char*>(base) + STATIC_ROWS_BYTES, static_cast<hipStream_t>(stream));
}
