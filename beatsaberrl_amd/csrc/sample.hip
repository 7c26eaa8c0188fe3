// Action epilogue on the (B, 29, K) fp32 logits: log-softmax, Gumbel-max sampling, summed
// log-probability and per-head entropy in one pass.
//
// Replaces the tail of the reference's `get_action_and_value` (python/policy.py:1467-1516):
//   logsm  = log_softmax(logits, -1)
//   action = argmax(logsm - log E), E ~ Exp(1); lanes past a head's gear count pinned to -inf
//   logp   = sum_heads logsm[action];  ent_h = -(exp(logsm) * logsm).sum(-1);  entropy = ent_h.sum(-1)
// The Exp(1) draws either come from the caller (`exp_noise`, e.g. torch's generator: then the
// result is a pure function of the inputs) or from a counter-based Philox4x32-10 stream keyed by
// (seed, offset) inside the kernel; a different stream than the caller's generator is the
// same accepted class of difference the reference documents for its own sampler change
// (python/policy.py:1476-1483).  The offset may live on the device (`offset_dev`, added to the
// host offset): a launch captured in a graph then draws fresh noise on every replay, provided
// something on the stream advances the counter between launches - bsrl_counter_add is that
// one-thread kernel (the role torch's graph-registered generator offset plays for the
// reference's captured rollout, python/rollout_graph.py:43-78).
//
// One thread per (env, head); a workgroup owns EPB envs and reduces the 29 per-head terms of
// each env in head order (a fixed order: results do not depend on the launch shape).
#include "bsrl_common.h"

namespace {

constexpr int EPB = 8;
constexpr int KMAX = 8;

struct SampleArgs {
    const float* logits; int64_t B; int n_heads, K;
    const int32_t* head_sizes; const float* exp_noise;
    uint64_t seed, offset; const uint64_t* offset_dev;
    const void* action_in; int action_in_u8;
    int64_t* action_out; float* logprob; float* entropy; float* ent_h; float* noise_out;
};

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11)
__device__ __forceinline__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1, n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
}
// 24 random bits -> u in (0, 1]; E = -log(u) >= 0 is Exp(1) (E == 0 with probability 2^-24,
// scoring +inf exactly as an E = 0 draw does in the reference).
__device__ __forceinline__ float exp1_from_bits(uint32_t x) { return -logf((float)((x >> 8) + 1u) * 5.9604644775390625e-8f); }

__global__ __launch_bounds__(256) void sample_heads_kernel(SampleArgs a) {
    __shared__ float s_lp[EPB][32], s_ent[EPB][32];
    const int tid = threadIdx.x;
    const int e = tid / 32, h = tid % 32;                    // 32 thread slots per env, n_heads <= 32 used
    const int64_t env = (int64_t)blockIdx.x * EPB + e;
    const bool live = env < a.B && h < a.n_heads;
    float lp = 0.f, ent = 0.f;
    if (live) {
        const int K = a.K;
        const int64_t row = env * a.n_heads + h;
        const float* x = a.logits + row * K;
        float v[KMAX];
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) { v[k] = k < K ? x[k] : -INFINITY; m = fmaxf(m, v[k]); }
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) s += k < K ? expf(v[k] - m) : 0.f;
        const float ls = logf(s);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) v[k] = (v[k] - m) - ls;          // log-softmax (lanes >= K: -inf, never read)
        int act;
        if (a.action_in) {
            act = a.action_in_u8 ? (int)static_cast<const uint8_t*>(a.action_in)[row]
                                 : (int)static_cast<const int64_t*>(a.action_in)[row];
            act = act < 0 ? 0 : (act >= K ? K - 1 : act);               // out-of-range actions are clamped into the row (documented in bsrl.h): never index out of it
        } else {
            const int nvalid = a.head_sizes ? a.head_sizes[h] : K;
            uint32_t r[8];
            if (!a.exp_noise) {
                // counter = (row, 2 * offset + block): 8 draws per row from two 128-bit blocks
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const uint64_t hi = (a.offset + (a.offset_dev ? *a.offset_dev : 0)) * 2u + (uint64_t)blk;
                    uint32_t c[4] = {(uint32_t)row, (uint32_t)((uint64_t)row >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
                    philox4x32_10(c, (uint32_t)a.seed, (uint32_t)(a.seed >> 32));
#pragma unroll
                    for (int j = 0; j < 4; ++j) r[4 * blk + j] = c[j];
                }
            }
            float best = -INFINITY; act = 0;
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
                if (k < K) {
                    const float E = a.exp_noise ? a.exp_noise[row * K + k] : exp1_from_bits(r[k]);
                    if (a.noise_out) a.noise_out[row * K + k] = E;
                    const float sc = k < nvalid ? v[k] - logf(E) : -INFINITY;
                    if (sc > best || (k == 0)) { best = sc; act = k; }   // first maximum wins
                }
            }
        }
        if (a.action_out) a.action_out[row] = act;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            if (k == act) lp = v[k];
            if (k < K) { const float p = expf(v[k]); ent -= p * v[k]; }
        }
        if (a.ent_h) a.ent_h[row] = ent;
    }
    s_lp[e][h] = lp; s_ent[e][h] = ent;
    __syncthreads();
    if (tid < EPB) {
        const int64_t env2 = (int64_t)blockIdx.x * EPB + tid;
        if (env2 < a.B) {
            float sl = 0.f, se = 0.f;
            for (int j = 0; j < a.n_heads; ++j) { sl += s_lp[tid][j]; se += s_ent[tid][j]; }
            a.logprob[env2] = sl;
            if (a.entropy) a.entropy[env2] = se;
        }
    }
}

__global__ void counter_add_kernel(uint64_t* ctr, uint64_t inc) { *ctr += inc; }

}  // namespace

extern "C" int bsrl_counter_add(uint64_t* counter, uint64_t inc, bsrl_stream stream) {
    if (!counter) BSRL_FAIL(BSRL_EINVAL, "bsrl_counter_add: null counter");
    hipLaunchKernelGGL(counter_add_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), counter, inc);
    BSRL_CHECK_LAUNCH("bsrl_counter_add");
    return BSRL_OK;
}

extern "C" int bsrl_sample_heads(const float* logits, int64_t B, int64_t n_heads, int64_t K,
                                 const int32_t* head_sizes, const float* exp_noise,
                                 uint64_t seed, uint64_t offset, const uint64_t* offset_dev,
                                 const void* action_in, int action_in_u8,
                                 int64_t* action_out, float* logprob, float* entropy, float* ent_h,
                                 float* noise_out, bsrl_stream stream) {
    if (!logits || !logprob) BSRL_FAIL(BSRL_EINVAL, "bsrl_sample_heads: null logits / logprob");
    if (B < 0 || n_heads < 1 || n_heads > 32 || K < 1 || K > KMAX)
        BSRL_FAIL(BSRL_EINVAL, "bsrl_sample_heads: need B >= 0, 1 <= n_heads <= 32, 1 <= K <= %d", KMAX);
    if (!action_in && !action_out) BSRL_FAIL(BSRL_EINVAL, "bsrl_sample_heads: sampling needs action_out");
    if (B == 0) return BSRL_OK;
    SampleArgs a{logits, B, (int)n_heads, (int)K, head_sizes, exp_noise, seed, offset, offset_dev, action_in, action_in_u8,
                 action_out, logprob, entropy, ent_h, noise_out};
    const dim3 grid((unsigned)((B + EPB - 1) / EPB)), block(256);
    hipLaunchKernelGGL(sample_heads_kernel, grid, block, 0, static_cast<hipStream_t>(stream), a);
    BSRL_CHECK_LAUNCH("bsrl_sample_heads");
    return BSRL_OK;
}
