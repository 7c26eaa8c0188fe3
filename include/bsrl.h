/* bsrl.h - C ABI of libbsrl_hip.so: the MI355X (gfx950) policy-forward kernels.
 *
 * Every entry point replaces one binding of the reference's two torch
 * extension modules (python/beat_arena_env/csrc/layer_norm.cu:733-749 and
 * python/beat_arena_env/csrc/fp16_gemm.cu:535-566) or one vendor call the
 * reference's op layer makes (python/fp16_linear.py:134-181).  The ABI is plain
 * C: raw device pointers, explicit sizes and strides (in ELEMENTS), a dtype
 * enum and a HIP stream handle.  No entry point allocates, synchronises or
 * keeps a pointer after it returns; all work is enqueued on `stream`
 * (NULL = the null stream) and is safe to capture in a HIP graph.
 *
 * Return value of every int function: 0 = enqueued; >0 = the shape / dtype /
 * alignment is not supported by this kernel set (the caller picks another
 * route, the reference signals the same with an empty list,
 * fp16_gemm.cu:346-357); <0 = invalid argument or HIP launch error, text in
 * bsrl_last_error() (thread-local).
 */
#ifndef BSRL_H
#define BSRL_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { BSRL_F32 = 0, BSRL_F16 = 1, BSRL_BF16 = 2 } bsrl_dtype;
typedef enum { BSRL_ACT_NONE = 0, BSRL_ACT_RELU = 1, BSRL_ACT_GELU = 2 } bsrl_act;

#define BSRL_OK 0
#define BSRL_UNSUPPORTED 1
#define BSRL_EINVAL (-1)
#define BSRL_ELAUNCH (-2)

#define BSRL_MASK_BIAS 16384.0f /* reference python/policy.py:428 */
#define BSRL_MAX_T 48
#define BSRL_MAX_LAYERS 8

typedef void* bsrl_stream; /* hipStream_t */

/* ABI version (bumped on any signature change). */
int bsrl_version(void);
/* Text of the last error on the calling thread ("" if none). */
const char* bsrl_last_error(void);

/* ---- LayerNorm ----------------------------------------------------------
 * Replaces layer_norm_cuda.ln_fwd (layer_norm.cu:530-561): y = LN(x) over the
 * last dim, fp32 weight/bias/statistics, x and y in `dtype`.  mean / rstd are
 * optional (NULL to skip) fp32 (rows,) outputs.  x, y contiguous (rows, d). */
int bsrl_ln_fwd(const void* x, const float* weight, const float* bias, void* y,
                float* mean, float* rstd, int64_t rows, int64_t d, float eps,
                int dtype, bsrl_stream stream);

/* Replaces layer_norm_cuda.ln_fwd_add (layer_norm.cu:563-643):
 * x = round(a + (b + b_bias)); y = LN(x) with statistics on the ROUNDED x.
 * b_bias is an optional fp32 (d,) vector (NULL = none). */
int bsrl_ln_fwd_add(const void* a, const void* b, const float* b_bias,
                    const float* weight, const float* bias, void* x, void* y,
                    float* mean, float* rstd, int64_t rows, int64_t d, float eps,
                    int dtype, bsrl_stream stream);

/* ---- Linear (+bias +activation +residual) --------------------------------
 * Replaces the vendor GEMM calls of python/fp16_linear.py:134-181 (addmm / mm /
 * _addmm_activation) and fp16_gemm.linear_relu_aux / bias_relu_
 * (fp16_gemm.cu:77-111, 404-497):
 *   y[r, m] = act( sum_k x[r, k] * w[m, k] + bias[m] ) + residual[r, m]
 * x (rows, K) row stride ldx; w (M, K) contiguous nn.Linear layout in `dtype`;
 * bias fp32 (M,) or NULL; residual in `dtype`, row stride ldr, or NULL;
 * y row stride ldy in `out_dtype` (same as dtype, or BSRL_F32).
 * If y2 != NULL, columns >= split go to y2[r * ldy2 + (m - split)] (fp32 when
 * out_dtype is F32) - used to split packed heads | value.
 * 16-bit dtypes run MFMA with fp32 accumulate; F32 runs an FMA kernel. */
int bsrl_linear(const void* x, int64_t ldx, const void* w, const float* bias,
                const void* residual, int64_t ldr, void* y, int64_t ldy,
                void* y2, int64_t ldy2, int64_t split,
                int64_t rows, int64_t K, int64_t M, int act, int dtype,
                int out_dtype, bsrl_stream stream);
/* bsrl_linear whose output rows are grouped: output row r is written at
 * y + (r / y_group_rows) * y_group_stride + (r % y_group_rows) * ldy (elements),
 * i.e. y is a (rows / y_group_rows, y_group_rows, M) slice of a larger tensor -
 * an encoder's tokens written straight into their rows of the (B, T, d) stream,
 * which replaces the reference's torch.cat of the token groups
 * (python/policy.py:1247-1249).  y_group_rows == 0: plain bsrl_linear.  No split
 * output in grouped form. */
int bsrl_linear_grouped(const void* x, int64_t ldx, const void* w, const float* bias,
                        const void* residual, int64_t ldr, void* y, int64_t ldy,
                        void* y2, int64_t ldy2, int64_t split,
                        int64_t rows, int64_t K, int64_t M, int act, int dtype, int out_dtype,
                        int64_t y_group_rows, int64_t y_group_stride, bsrl_stream stream);
/* Two Linears with a ReLU between them in one launch: y = relu(x W1^T + b1) W2^T + b2 - a token encoder of the
 * policy (python/policy.py:1224-1249, `_seq` / `_run` python/policy.py:76-145: Linear(in, d) ReLU Linear(d, d) through
 * fp16_linear_relu and fp16_linear, python/fp16_linear.py:134-181), the hidden rows never written.  x (rows, K1) with
 * row stride ldx, w1 (d, K1), w2 (d, d) in `dtype` (nn.Linear layout), b1 / b2 fp32 (d); y and its row grouping as
 * in bsrl_linear_grouped.  Bit for bit what bsrl_linear(act = ReLU) followed by bsrl_linear_grouped gives.  16-bit
 * dtypes, K1 = 64, d = 128 / 192, 16-byte aligned rows; BSRL_UNSUPPORTED otherwise (run the two Linears). */
int bsrl_mlp2(const void* x, int64_t ldx, const void* w1, const float* b1, int64_t K1, const void* w2,
              const float* b2, void* y, int64_t ldy, int64_t rows, int64_t d, int dtype,
              int64_t y_group_rows, int64_t y_group_stride, bsrl_stream stream);

/* ---- Short-sequence masked multi-head attention ----------------------------
 * Replaces fp16_gemm.attn29_fwd (small_attn.cu:515-536) and the SDPA / fp32
 * fallbacks it shadows (python/policy.py:684-690):
 *   out[b, tq, h*dh:(h+1)*dh] = softmax_k(q.k / sqrt(dh) + key_bias[b, k]) v
 * q (B, TQ, H*dh): element (b,t,c) at q[b*q_bs + t*q_rs + c]; likewise k, v
 * (B, T, H*dh) with their own strides, so q|k|v may be views of one packed
 * projection.  The key mask is either key_bias (B, T) in `dtype` (additive,
 * 0 or -2^14) or n_valid (B,) int32 (keys 0..n_valid[b] attendable); pass one,
 * or neither for no mask.  out (B, TQ, H*dh) contiguous in `dtype`.
 * T <= 48, TQ <= T, dh in {32, 48} (16-bit) or any dh <= 64 (F32). */
int bsrl_attn_fwd(const void* q, int64_t q_bs, int64_t q_rs,
                  const void* k, int64_t k_bs, int64_t k_rs,
                  const void* v, int64_t v_bs, int64_t v_rs,
                  const void* key_bias, const int32_t* n_valid, void* out,
                  int64_t B, int64_t T, int64_t TQ, int64_t H, int64_t dh,
                  int dtype, bsrl_stream stream);

/* Backward of bsrl_attn_fwd; replaces fp16_gemm.attn29_bwd(q, k, v, bias, dout,
 * dq, dk, dv) (small_attn.cu:345-463, 539-571), which likewise writes the three
 * gradients into caller views (column slices of one packed q|k|v gradient).
 * The probabilities are recomputed from q, k and the mask as the forward does:
 *   dP = dO V^T, dS = P * (dP - rowsum(P * dP)), dQ = dS K / sqrt(dh),
 *   dK = dS^T Q / sqrt(dh), dV = P^T dO        (fp32 scores / softmax / sums)
 * q, k, v, key_bias, n_valid, B, T, TQ, H, dh: as bsrl_attn_fwd.  dout (B, TQ, H*dh),
 * dq (B, TQ, H*dh), dk, dv (B, T, H*dh): element (b, t, c) at p[b*bs + t*rs + c],
 * each with its own strides; masked keys get dk = dv = 0.  16-bit: dh in {32, 48},
 * 16-byte aligned input rows, 8-byte aligned gradient rows; F32: dh <= 48. */
int bsrl_attn_bwd(const void* q, int64_t q_bs, int64_t q_rs,
                  const void* k, int64_t k_bs, int64_t k_rs,
                  const void* v, int64_t v_bs, int64_t v_rs,
                  const void* key_bias, const int32_t* n_valid,
                  const void* dout, int64_t do_bs, int64_t do_rs,
                  void* dq, int64_t dq_bs, int64_t dq_rs,
                  void* dk, int64_t dk_bs, int64_t dk_rs,
                  void* dv, int64_t dv_bs, int64_t dv_rs,
                  int64_t B, int64_t T, int64_t TQ, int64_t H, int64_t dh,
                  int dtype, bsrl_stream stream);

/* ---- Fused FFN ------------------------------------------------------------
 * Replaces fp16_gemm.ffn_fused (fused_ffn.cu:551-619):
 *   xo = x + act(h2 w0^T + b0) w2^T + b2 ;  ho = LN_next(xo) if ln_w != NULL
 * x, h2, xo, ho (rows, d) contiguous in `dtype` (16-bit only); w0 (F, d),
 * w2 (d, F) in `dtype`; b0, b2, ln_w, ln_b fp32.  The hidden never reaches
 * memory.  d in {128, 192, 256, 384}, F = multiple of 32. */
int bsrl_ffn_fused(const void* x, const void* h2, const void* w0, const float* b0,
                   const void* w2, const float* b2, const float* ln_w,
                   const float* ln_b, float eps, void* xo, void* ho,
                   int64_t rows, int64_t d, int64_t F, int act, int dtype,
                   bsrl_stream stream);
/* Mirrors fp16_gemm.ffn_fused_supported (fused_ffn.cu:509-525): 1 if the
 * (d, F, dtype) combination has a kernel. */
int bsrl_ffn_fused_supported(int64_t d, int64_t F, int dtype);
/* The same operation (fp16_gemm.ffn_fused, fused_ffn.cu:551-619; same rounding points) from a
 * weight image in MFMA fragment order, for d in {128, 192, 256, 384} and F a multiple of 32 with
 * F/16 >= 10 / 7 / 6 / 5 (d = 128 / 192 / 256 / 384): the weights stream straight into LDS and a
 * wave owns 32 rows.  bsrl_ffn_pack writes the image (bsrl_ffn_pack_size bytes, 16-byte aligned; 0 =
 * unsupported shape) from w0 (F, d) and w2 (d, F) in `dtype` and the fp32 biases - once per
 * weight update, like the 16-bit replicas the reference keeps (python/fp16_linear.py:150-192);
 * bsrl_ffn_packed is bsrl_ffn_fused with the image in place of w0, b0, w2, b2.  x, h2, xo, ho
 * (rows, d) contiguous in `dtype`, 8-byte aligned (d = 384: 16-byte).  hid, if not NULL, receives the activated
 * hidden (rows, F) in `dtype` exactly as the down-projection consumed it - what the reference's
 * kernel returns for the backward (fused_ffn.cu:551-619, `hid`; its ReLU mask is hid > 0). */
int64_t bsrl_ffn_pack_size(int64_t d, int64_t F, int dtype);
int bsrl_ffn_pack(const void* w0, const float* b0, const void* w2, const float* b2,
                  int64_t d, int64_t F, int dtype, void* image, bsrl_stream stream);
int bsrl_ffn_packed(const void* image, const void* x, const void* h2, const float* ln_w,
                    const float* ln_b, float eps, void* xo, void* ho, void* hid, int64_t rows,
                    int64_t d, int64_t F, int act, int dtype, bsrl_stream stream);
/* The tail of a block from the attention output on, in one kernel (d = 384, where the per-op route
 * runs the block as separate launches):
 *   x1 = x + att Wo^T + bo            Block.forward's output projection + residual (python/policy.py:650-662)
 *   h2 = LayerNorm(x1; ln2_w, ln2_b)  its ln_ffn (python/policy.py:663-672, layer_norm.cu:14-21)
 *   xo = x1 + act(h2 W0^T + b0) W2^T + b2,  ho = LayerNorm(xo; ln_w, ln_b) if ln_w   (bsrl_ffn_packed)
 * with the rounding points of the separate launches (x1, h2, hidden, xo, ho rounded once each; fp32
 * accumulation and statistics), x1 and h2 never leaving the registers.  With n_next > 0 (a multiple
 * of 64, at most 3 d) the NEXT block's packed projection comes out of the same launch:
 *   qo = ho Wn^T + bn                 the q|k|v Linears of Block.forward (python/policy.py:541-560)
 * (rows, n_next), rounded once, ho's fragments taken from the registers; ho itself is then written only
 * if the pointer is given.  bsrl_proj_ffn_pack writes the image (bsrl_proj_ffn_pack_size bytes,
 * 16-byte aligned; 0 = unsupported shape) from wo (d, d), w0 (F, d), w2 (d, F), wn (n_next, d; NULL
 * when n_next = 0) in `dtype` and the fp32 biases.  att, x, xo, ho (rows, d), qo (rows, n_next)
 * contiguous in `dtype`, 16-byte aligned; ln2_w / ln2_b required; ln_w / ln_b together; without a
 * projection behind, ho goes with them. */
int64_t bsrl_proj_ffn_pack_size(int64_t d, int64_t F, int64_t n_next, int dtype);
int bsrl_proj_ffn_pack(const void* wo, const float* bo, const void* w0, const float* b0,
                       const void* w2, const float* b2, const void* wn, const float* bn,
                       int64_t n_next, int64_t d, int64_t F, int dtype, void* image,
                       bsrl_stream stream);
int bsrl_proj_ffn_packed(const void* image, const void* att, const void* x, const float* ln2_w,
                         const float* ln2_b, float eps2, const float* ln_w, const float* ln_b,
                         float eps, void* xo, void* ho, void* qo, int64_t n_next, int64_t rows,
                         int64_t d, int64_t F, int act, int dtype, bsrl_stream stream);
/* The last phase of that kernel alone, for the first block of a stack (d = 384):
 *   ho = LayerNorm(x; ln_w, ln_b)     Block.forward's ln_attn (python/policy.py:541, layer_norm.cu:14-21)
 *   qo = ho Wn^T + bn                 its packed q|k|v Linears (python/policy.py:541-560)
 * one launch, ho's fragments taken from the registers (ho itself written only if the pointer is
 * given).  n_next a multiple of 64 in [192, 3 d]; image (bsrl_ln_proj_pack_size bytes, 16-byte
 * aligned; 0 = unsupported) from wn (n_next, d) in `dtype` and bn fp32.  x, ho (rows, d), qo
 * (rows, n_next) contiguous in `dtype`, 16-byte aligned. */
int64_t bsrl_ln_proj_pack_size(int64_t d, int64_t n_next, int dtype);
int bsrl_ln_proj_pack(const void* wn, const float* bn, int64_t n_next, int64_t d, int dtype,
                      void* image, bsrl_stream stream);
int bsrl_ln_proj_packed(const void* image, const void* x, const float* ln_w, const float* ln_b,
                        float eps, void* ho, void* qo, int64_t n_next, int64_t rows, int64_t d,
                        int dtype, bsrl_stream stream);

/* ---- Config-model tokenizer -----------------------------------------------
 * The benchmark configs' "linear embedding": token 0 = Wp obs[:, :prop_dim] +
 * bp, token j = Wo obs[:, prop_dim + (j-1)*obj_dim : ...] + bo
 * (the reference's encoder stage, python/policy.py:1224-1249, reduced to one
 * Linear per token type).  obs (B, obs_ld) in obs_dtype (F32 or `dtype`),
 * rounded once to `dtype` like python/policy.py:1200-1209; wp (d, prop_dim),
 * wo (d, obj_dim) in `dtype`; tokens (B, T, d) contiguous in `dtype`. */
int bsrl_cfg_embed(const void* obs, int64_t obs_ld, int obs_dtype,
                   const void* wp, const float* bp, const void* wo, const float* bo,
                   void* tokens, int64_t B, int64_t T, int64_t d,
                   int64_t prop_dim, int64_t obj_dim, int dtype, bsrl_stream stream);

/* ---- Whole config-model forward in one persistent kernel -------------------
 * Replaces NotePolicy.forward_stacked (python/policy.py:1179-1344) for the
 * benchmark-config model: obs -> logits (B, 29*n_gears) fp32 + value (B,) fp32.
 * `packed` is the weight image written by bsrl_cfg_pack() for the same
 * (n_layers, d, n_heads, ffn, T) - the analogue of the reference's flat fp16
 * replica buffer (python/fp16_linear.py:249-346): rebuilt after each optimizer
 * step, its address must not move while a captured graph replays. */
typedef struct {
    int32_t n_layers, d, n_heads, ffn, T, n_gears, act, final_ln;
    int32_t prop_dim, obj_dim, dtype, flags;      /* flags: 0, or BSRL_CFG_NO_PACK | BSRL_CFG_NO_LATENCY */
} bsrl_cfg_desc;
/* bsrl_cfg_forward: keep every env in a tile of its own (see below). */
#define BSRL_CFG_NO_PACK 1
/* bsrl_cfg_forward: never take the latency form.  By default a batch of at
 * most 4 envs per CU (B <= 1024 on an MI355X) runs as ONE persistent launch
 * whatever the workspace: one env per wave (1..4 working waves per workgroup,
 * as few as the batch allows), the weight image streamed straight into a
 * 14-slot LDS ring 13 stages ahead, the next stage's fragments fetched into
 * registers while the current one is computed.  At such sizes a forward is one
 * workgroup's walk through the ~100 stages of the image and its time is what a
 * lone CU takes to pull 0.9 MB and to run the dependent chain of each stage
 * (B = 1: 33 us against 52 us for the throughput forms).  The output bits are
 * those of the other forms (tested), so an env's result does not change with
 * the batch it is in.  Shapes whose vectors + ring exceed a workgroup's LDS
 * (n_layers * (9 d + ffn) floats + 112 KB > 158 KB) always take the other forms. */
#define BSRL_CFG_NO_LATENCY 2

/* fp32 master parameter pointers of one transformer block, in the reference's
 * registration order (python/policy.py:492-522); device memory. */
typedef struct {
    const float *ln_attn_w, *ln_attn_b, *q_w, *q_b, *k_w, *k_b, *v_w, *v_b,
        *out_w, *out_b, *ln_ffn_w, *ln_ffn_b, *ffn0_w, *ffn0_b, *ffn2_w, *ffn2_b;
} bsrl_block_params;

/* fp32 master parameter pointers in state_dict order (device memory). */
typedef struct {
    const float *prop_w, *prop_b, *obj_w, *obj_b;
    bsrl_block_params blk[BSRL_MAX_LAYERS];
    const float *final_ln_w, *final_ln_b, *heads_w, *heads_b;
} bsrl_cfg_params;

/* Bytes of the packed image for `desc`, or 0 if the fused kernel does not
 * support this shape (use the per-op entry points instead). */
int64_t bsrl_cfg_pack_size(const bsrl_cfg_desc* desc);
/* One cast+permute pass: fp32 masters -> packed 16-bit MFMA-fragment-major
 * image (the analogue of fp16_linear.flat_refresh, fp16_linear.py:241-246). */
int bsrl_cfg_pack(const bsrl_cfg_desc* desc, const bsrl_cfg_params* params,
                  void* packed, bsrl_stream stream);
/* Bytes of scratch the pruned form of bsrl_cfg_forward needs for B envs
 * (768 B per env for the parked rows + 16 B per env + 16 B for the tile table of
 * the packed launch), or 0 if the shape is unsupported. */
int64_t bsrl_cfg_workspace_size(const bsrl_cfg_desc* desc, int64_t B);
/* obs (B, obs_ld) F32 or 16-bit; n_valid (B,) int32 or NULL (all valid).
 * workspace == NULL (or smaller than bsrl_cfg_workspace_size): ONE persistent
 * kernel computes every token of every block.  With a workspace: final-block
 * query pruning, the reference's n_queries path (python/policy.py:533-539,
 * :1302-1305; exact, masking is key-side only): the tokenizer, blocks 0..L-2
 * and the last block's attention run on whole envs, each env's token-0 row is
 * parked in the workspace, and the last block's output projection + FFN and
 * the heads run on those rows, 16 envs per MFMA tile.  That is ONE launch:
 * every workgroup runs the tail of the envs it parked itself, whenever 64 of
 * them wait and once more at the end; no workgroup waits for another.  (Models
 * whose weight ring cannot live in LDS twice per CU - vectors + 96 KB beyond
 * 160 KB - run the tail as a second launch.)  With n_valid given and the full
 * workspace, short envs share 16-row tiles under a block-diagonal key mask:
 * two of 5..8 tokens (n_valid 4..7) at rows 0 / 8; one of at most 4 tokens
 * (n_valid <= 3) at rows 12.. behind one of 9..12 tokens, or four of them at
 * rows 0 / 4 / 8 / 12.  Up to 16384 envs every workgroup derives its tiles
 * from the key counts itself (class prefixes in LDS); beyond, a small kernel
 * builds the tile table in the workspace on the stream first.  Padded rows are
 * what the reference computes and discards (python/policy.py:1257-1260 masks
 * them key-side), and an env's output bits are the same packed or alone.
 * desc->flags = BSRL_CFG_NO_PACK keeps one env per tile; a workspace of only
 * 768 B per env, or an n_valid that is not 16-byte aligned, does too.
 * Batches of at most 4 envs per CU take the latency form (one launch, no
 * workspace use) unless BSRL_CFG_NO_LATENCY is set.  All forms give the same
 * output bits. */
int bsrl_cfg_forward(const bsrl_cfg_desc* desc, const void* packed,
                     const void* obs, int64_t obs_ld, int obs_dtype,
                     const int32_t* n_valid, float* logits, float* value,
                     int64_t B, void* workspace, int64_t workspace_bytes,
                     bsrl_stream stream);

/* bsrl_cfg_forward for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference (whose ops allocate their outputs,
 * layer_norm.cu:545-547).  Same arguments and results as bsrl_cfg_forward with a
 * full workspace - the same kernels on the same launch shapes, so the same
 * output bits - but the parked rows (and, beyond the in-kernel tile table's
 * batch limit, the tile table) live in a device array built into the library
 * (BSRL_CFG_STATIC_MAX_ENVS * 784 + 16 bytes, held on every GPU the library is
 * used on until the process ends) instead of a caller workspace; the call
 * allocates and frees nothing.  Batches of at most 4 envs per CU take the
 * latency form here too, which uses no scratch at all.  B >
 * BSRL_CFG_STATIC_MAX_ENVS is an error (BSRL_EINVAL); ffn not a multiple of 64
 * returns BSRL_UNSUPPORTED.  Every call on one GPU shares that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race -
 * serialise them or use bsrl_cfg_forward with one workspace per stream.
 * Nothing in the array has to be cleared between calls.  The FIRST call on a
 * device takes the array's address (hipGetSymbolAddress: the runtime loads
 * the code object) and may raise a kernel's LDS limit (hipFuncSetAttribute):
 * make it outside stream capture; later calls only launch and are capturable
 * (tests/test_zz_no_alloc.py replays one from a graph). */
#define BSRL_CFG_STATIC_MAX_ENVS 16384
int bsrl_cfg_forward_static(const bsrl_cfg_desc* desc, const void* packed,
                            const void* obs, int64_t obs_ld, int obs_dtype,
                            const int32_t* n_valid, float* logits, float* value,
                            int64_t B, bsrl_stream stream);

/* ---- NotePolicy front end --------------------------------------------------
 * One pass over the (B, 630) observation that writes every encoder input and
 * the additive key bias.  Replaces the preamble of the reference forward
 * (python/policy.py:1199-1260): the one-time rounding of the obs to the stream
 * dtype (:1199-1209), NotePolicy._split (:1099-1105), _note_geo (:329-404,
 * fp32 arithmetic on the rounded lanes, one rounding on store), the hand / side
 * one-hot concatenations (:1231-1246) and the key-bias build (:1257-1260).
 * obs (B, obs_ld) in obs_dtype = F32 or `dtype`; saber_idx: 94 obs lanes (left
 * hand's 47, right hand's 47; the reference's `_saber_idx` buffer), body_idx:
 * 93 obs lanes (torso 29, left leg 32, right leg 32; `_body_idx`), both int32 on
 * the device.  Outputs, contiguous, in `dtype`: saber_in (B, 2, 49), torso_in
 * (B, 29), leg_in (B, 2, 34), note_in (B, 24, note_geo ? 40 : 18), key_bias
 * (B, 29) = 0 for the 5 lead tokens, (mask - 1) * 16384 for the 24 slots. */
int bsrl_note_frontend(const void* obs, int64_t obs_ld, int obs_dtype,
                       const int32_t* saber_idx, const int32_t* body_idx,
                       int note_geo, int flux, float z_asinh,
                       void* saber_in, void* torso_in, void* leg_in, void* note_in, void* key_bias,
                       int64_t B, int dtype, bsrl_stream stream);

/* The same pass with every encoder-input row written at a pitch of 64 elements,
 * zero past its natural width: saber_in (B, 2, 64), torso_in (B, 64), leg_in
 * (B, 2, 64), note_in (B, 24, 64).  The first Linear of each encoder MLP
 * (python/policy.py:1231-1246) then runs as a K = 64 GEMM against a weight whose
 * columns are zero-padded the same way; the zero lanes add nothing to the fp32
 * accumulators, so the tokens are the ones the unpadded route produces. */
int bsrl_note_frontend_padded(const void* obs, int64_t obs_ld, int obs_dtype,
                              const int32_t* saber_idx, const int32_t* body_idx,
                              int note_geo, int flux, float z_asinh,
                              void* saber_in, void* torso_in, void* leg_in, void* note_in, void* key_bias,
                              int64_t B, int dtype, bsrl_stream stream);

/* ---- Action epilogue ---------------------------------------------------------
 * log-softmax + Gumbel-max sampling + summed log-probability + per-head entropy
 * on the fp32 logits (B, n_heads, K), K <= 8, n_heads <= 32.  Replaces the tail
 * of get_action_and_value (python/policy.py:1467-1516).
 * Sampling (action_in == NULL): action = argmax_k(logsm[k] - log E[k]); lanes
 * k >= head_sizes[h] (int32 (n_heads), NULL = all K) score -inf
 * (python/policy.py:1487-1491).  E (B, n_heads, K) fp32 Exp(1) draws come from
 * exp_noise, or, when it is NULL, from Philox4x32-10 with key = seed and
 * counter = (row, 2 * offset + block) inside the kernel (row = env * n_heads +
 * head; draw k of a row is word k & 3 of block k >> 2, mapped to
 * E = -log(((word >> 8) + 1) * 2^-24)); offset_dev, if not NULL, points to a
 * device uint64 added to `offset` when the kernel runs, so a launch captured in
 * a graph draws fresh noise on each replay once bsrl_counter_add follows it on
 * the stream (the part torch's graph-registered generator offset plays in the
 * reference's captured rollout, python/rollout_graph.py:43-78).  noise_out, if
 * not NULL, receives the E used.  Evaluation (action_in != NULL, int64 or uint8 when action_in_u8):
 * no sampling; action_out may be NULL.  A given action outside [0, K) is clamped into the row (the
 * reference's torch.gather would raise): validate on the host where that matters - no entry point
 * synchronises, so the kernel cannot report it.
 * Outputs: action_out (B, n_heads) int64; logprob (B); entropy (B) or NULL;
 * ent_h (B, n_heads) or NULL. */
int bsrl_sample_heads(const float* logits, int64_t B, int64_t n_heads, int64_t K,
                      const int32_t* head_sizes, const float* exp_noise,
                      uint64_t seed, uint64_t offset, const uint64_t* offset_dev,
                      const void* action_in, int action_in_u8,
                      int64_t* action_out, float* logprob, float* entropy, float* ent_h,
                      float* noise_out, bsrl_stream stream);
/* *counter += inc, one thread, on `stream` (ordered after the launches before it). */
int bsrl_counter_add(uint64_t* counter, uint64_t inc, bsrl_stream stream);

/* ---- Transformer block stack in one persistent kernel ------------------------
 * Replaces the block loop of NotePolicy._forward_stacked (python/policy.py:
 * 1262-1306): every Block.forward (python/policy.py:524-715) of the stack -
 * LayerNorm, q|k|v projection, attention with the additive key bias, output
 * projection + residual, LayerNorm, FFN + residual - with the residual stream
 * held in fp32 registers from the first block to the last.
 * Shapes: T <= 32 tokens per env, d = 128 (4 heads x 32) or 192 (4 x 48), ffn a
 * multiple of 32, act RELU or GELU, dtype F16 or BF16.  n_queries > 0 restricts
 * the LAST block to its first n_queries (<= 16) rows, the reference's n_queries
 * path (python/policy.py:533-539; exact: masking is key-side only).
 * `packed` = image written by bsrl_blocks_pack for the same desc (rebuild after
 * each optimizer step; the address must not move under a captured graph).
 * x_in (B, T, d), key_bias (B, T) in `dtype`, contiguous.  x_out: (B, n_queries, d)
 * when n_queries > 0, else (B, T, d).  x_res (B, T, d) or NULL: with n_queries > 0,
 * the stream entering the last block (what the reference's critic reads,
 * python/policy.py:1296-1301). */
typedef struct {
    int32_t n_layers, d, n_heads, ffn, T, act, n_queries, dtype;
} bsrl_blocks_desc;
typedef struct {
    bsrl_block_params blk[BSRL_MAX_LAYERS];
} bsrl_blocks_params;
/* Bytes of the packed image, or 0 if the shape is unsupported. */
int64_t bsrl_blocks_pack_size(const bsrl_blocks_desc* desc);
int bsrl_blocks_pack(const bsrl_blocks_desc* desc, const bsrl_blocks_params* params,
                     void* packed, bsrl_stream stream);
int bsrl_blocks_forward(const bsrl_blocks_desc* desc, const void* packed,
                        const void* x_in, const void* key_bias,
                        void* x_res, void* x_out, int64_t B, bsrl_stream stream);

/* ---- Critic attention pool (one query per env) ----------------------------------
 * The attention of the reference's adapool critic (NotePolicy._critic, python/policy.py:1346-1403: critic_ln, k|v
 * projection of all T tokens, 1-query multi-head attention) without the (B T, 2d) keys and values: with one query
 * the projections commute with the pool.  Given qk (B, H, d) with qk[b, h] = Wk[h rows]^T q[b, h cols] this computes
 *   hv_j = LN(x_res[b, j]) (rounded to `dtype`), p[h] = softmax_j(hv_j . qk[b, h] / sqrt(d / H) + key_bias[b, j]),
 *   pooled[b, h, :] = sum_j p[h][j] hv_j
 * (q_h . bk_h is constant over j and cancels; the caller finishes a_h = Wv[h rows] pooled_h + bv_h because the
 * probabilities sum to 1).  x_res (B, T, d), qk (B, H, d), key_bias (B, T) or NULL, pooled (B, H, d): contiguous in
 * `dtype`; ln_weight / ln_bias fp32 (d).  16-bit dtypes, T <= 32, H <= 16, d = 128 / 192 / 256 (the scores and the
 * pool run as MFMAs, one wave per env); BSRL_UNSUPPORTED beyond - the caller then takes the k|v projection and
 * bsrl_attn_fwd. */
int bsrl_critic_pool(const void* x_res, const float* ln_weight, const float* ln_bias, float eps,
                     const void* qk, const void* key_bias, void* pooled,
                     int64_t B, int64_t T, int64_t d, int64_t H, int dtype, bsrl_stream stream);

/* ---- LayerNorm backward --------------------------------------------------------
 * Replaces layer_norm_cuda.ln_bwd(x, dy, w, mean, rstd, gx=None, want_dbb=False)
 * (python/beat_arena_env/csrc/layer_norm.cu:645-729), the backward of both
 * _LnFn and _LnAddFn (python/fused_ln.py:56-112).  x, dy, gx (NULL = none),
 * dx: (rows, d) contiguous in `dtype`; weight (d), mean / rstd (rows) fp32 (the
 * forward's statistics).  With g = dy * w, xhat = (x - mean) * rstd:
 *   dx = (g - mean_d(g) - xhat * mean_d(g * xhat)) * rstd + gx   (one rounding)
 *   dw = sum_rows dy * xhat, db = sum_rows dy                      (fp32, (d))
 *   dbb (NULL = skip) = sum_rows of the stored dx: the folded-bias gradient of
 *   ln_fwd_add's b_bias (python/fused_ln.py:96-106)
 * Column sums are reproducible run to run (fixed-order partials, no atomics).
 * workspace: caller-owned scratch of bsrl_ln_bwd_workspace_size(d) bytes, 16-byte
 * aligned, overwritten by each call.  Same shape limits as the forward up to
 * d = 1024 (fp32) / 2048 (16-bit); returns BSRL_UNSUPPORTED beyond. */
int64_t bsrl_ln_bwd_workspace_size(int64_t d);
int bsrl_ln_bwd(const void* x, const void* dy, const float* weight,
                const float* mean, const float* rstd, const void* gx,
                void* dx, float* dw, float* db, float* dbb, void* workspace,
                int64_t rows, int64_t d, int dtype, bsrl_stream stream);

/* ---- Data gradient through a ReLU -------------------------------------------------
 * Replaces fp16_gemm.dgrad_drelu(g, w, mask) (python/beat_arena_env/csrc/
 * fp16_gemm.cu:479-518; caller python/fp16_linear.py:719-727, 1241-1245):
 *   y[r, m] = (sum_k x[r, k] * w[m, k]) * [gate[r, m] > 0]
 * i.e. the data gradient of the Linear AFTER a ReLU (x = its output gradient,
 * w = its weight transposed, (M, K) contiguous) masked by that ReLU in the GEMM
 * epilogue; gate = the ReLU's forward output (the saved hidden), which stands in
 * for the reference's bitmask.  x (rows, K) pitch ldx, gate / y (rows, M) pitches
 * ldgate / ldy, all in `dtype`; same kernels and shape coverage as bsrl_linear. */
int bsrl_linear_gated(const void* x, int64_t ldx, const void* w, const void* gate, int64_t ldgate,
                      void* y, int64_t ldy, int64_t rows, int64_t K, int64_t M, int dtype,
                      bsrl_stream stream);

/* gm = g * [y > 0]: the gradient through a ReLU from its saved forward output
 * (fp16_gemm.relu_bwd, python/beat_arena_env/csrc/fp16_gemm.cu:113-187; the bias
 * gradient the reference folds into that pass comes from bsrl_wgrad here).
 * g, y, out: (rows, d) in `dtype` with row pitches in elements; out may alias g. */
int bsrl_relu_bwd(const void* g, int64_t ldg, const void* y, int64_t ldy, void* out, int64_t ldo,
                  int64_t rows, int64_t d, int dtype, bsrl_stream stream);

/* ---- Linear weight / bias gradient -----------------------------------------------
 * Replaces fp16_gemm.wgrad(dy, x) -> dW and wgrad_bgrad(dy, x) -> [dW, db]
 * (python/beat_arena_env/csrc/fp16_gemm.cu:189-277, 404-476; callers
 * python/fp16_linear.py:442-458):
 *   dW[m, k] = sum_r dy[r, m] * x[r, k]   (fp32, (M, K) contiguous)
 *   db[m]    = sum_r dy[r, m]              (fp32 (M), NULL = skip)
 * dy (rows, M) row pitch lddy, x (rows, K) row pitch ldx, both F16 or BF16 (the
 * fp32 stream uses the vendor GEMM, as the reference does); fp32 accumulation
 * on MFMA, reproducible run to run (row splits folded in a fixed order).
 * workspace: caller-owned scratch of bsrl_wgrad_workspace_size(M, K) bytes,
 * overwritten by each call. */
int64_t bsrl_wgrad_workspace_size(int64_t M, int64_t K);
int bsrl_wgrad(const void* dy, int64_t lddy, const void* x, int64_t ldx,
               float* dw, float* db, void* workspace,
               int64_t rows, int64_t M, int64_t K, int dtype, bsrl_stream stream);

/* ---- Value-residual mix -------------------------------------------------------
 * out = a * v + b * v0: what every block after the first does to its attention
 * values under the reference's value_residual option (fp16_linear.vres_mix,
 * python/fp16_linear.py:1002-1006; call site python/policy.py:568-611).  fp32
 * arithmetic ((v * a) rounded to fp32, then + v0 * b fused), one rounding to
 * `dtype`; exactly v at (a, b) = (1, 0).  a, b: device pointers to the learned
 * fp32 scalars (no host read).  v, v0, out: (rows, d) with row pitches ldv,
 * ldv0, ldo in elements (views into packed q|k|v buffers); out may alias v. */
int bsrl_vres_mix(const void* v, int64_t ldv, const void* v0, int64_t ldv0,
                  const float* a, const float* b, void* out, int64_t ldo,
                  int64_t rows, int64_t d, int dtype, bsrl_stream stream);

/* ---- SimBaV2 readout stages ----------------------------------------------------
 * The fp32 row work between the three GEMMs of the reference's hyperspherical
 * trunk (NotePolicy._trunk_v2, python/policy.py:1140-1155; l2n = F.normalize
 * with eps 1e-6, :742-744), with l2n(x) = x / max(|x|_2, 1e-6), t (rows, D) in
 * `dtype` (a GEMM output), s (D) fp32 scaler and c its constant factor:
 *   BSRL_HS_SCALE_L2N : x = l2n(t * (s * c))      -> x32_out (rows, D) fp32 and,
 *                       if x_out is not NULL, the same rounded to `dtype`
 *   BSRL_HS_SCALE_RELU: x_out = relu(t * (s * c))  rounded to `dtype`
 *   BSRL_HS_L2N_LERP  : y = l2n(t); z = l2n(x32_in + (s * c) * (y - x32_in));
 *                       x_out = sqrt(D) * z rounded to `dtype` */
#define BSRL_HS_SCALE_L2N 0
#define BSRL_HS_SCALE_RELU 1
#define BSRL_HS_L2N_LERP 2
int bsrl_hsphere(int op, const void* t, const float* s, float c,
                 const float* x32_in, float* x32_out, void* x_out,
                 int64_t rows, int64_t D, int dtype, bsrl_stream stream);

/* out[r] = sum_i softmax(logits[r, :])_i * centers[i]: the expectation that ends the HL-Gauss critic,
 * `torch.softmax(logits, -1) @ self.value_centers` (python/policy.py:1394-1403), as one kernel on the
 * fp32 bin logits instead of a softmax pass, a gemv and their temporaries.  logits (rows, n) fp32
 * contiguous, centers (n) fp32, out (rows) fp32; fp32 arithmetic, max-subtracted. */
int bsrl_softmax_expect(const float* logits, const float* centers, float* out, int64_t rows, int64_t n,
                        bsrl_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* BSRL_H */
