// Config-model tokenizer: obs -> (B, T, d) tokens, one Linear per token type.
//
// token 0 = Wp . obs[0:prop_dim] + bp ; token j = Wo . obs[prop_dim + (j-1)*obj_dim : ...] + bo.
// A workgroup owns EPB = 4 envs: their obs rows are rounded once to the stream
// dtype (the reference rounds the obs once on entry to the fp16 stream,
// python/policy.py:1200-1209) and parked in LDS as fp32; thread f owns output
// feature f and walks its two weight rows once for all 4 envs x T tokens
// (4 + 4*(T-1) fp32 accumulators), so the weights are read once per workgroup.
// ~2% of the forward's MACs; the fused whole-forward kernel does this step on
// the matrix cores instead.
#include "bsrl_common.h"

namespace {

constexpr int EPB = 4;

struct EmbedArgs {
    const void* obs; int64_t obs_ld; int obs_f32;
    const void* wp; const float* bp; const void* wo; const float* bo;
    void* tokens; int64_t B; int T, d, prop_dim, obj_dim;
};

template <typename IO> struct EmbIO;
template <> struct EmbIO<F32IO> {
    static __device__ __forceinline__ float ld(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
    static __device__ __forceinline__ float round(float v) { return v; }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
};
template <typename DT> struct EmbIO16 {
    static __device__ __forceinline__ float ld(const void* p, int64_t i) { return DT::to_f(static_cast<const u16*>(p)[i]); }
    static __device__ __forceinline__ float round(float v) { return DT::to_f(DT::from_f(v)); }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { static_cast<u16*>(p)[i] = DT::from_f(v); }
};
template <> struct EmbIO<F16> : EmbIO16<F16> {};
template <> struct EmbIO<BF16> : EmbIO16<BF16> {};

template <typename IO, int NMAX>   // NMAX >= T - 1 object tokens
__global__ __launch_bounds__(256) void cfg_embed_kernel(EmbedArgs a) {
    extern __shared__ float so[];                      // [EPB][obs_dim]
    typedef EmbIO<IO> io;
    const int nobj = a.T - 1;
    const int obs_dim = a.prop_dim + nobj * a.obj_dim;
    const int64_t b0 = (int64_t)blockIdx.x * EPB;
    for (int i = threadIdx.x; i < EPB * obs_dim; i += blockDim.x) {
        const int e = i / obs_dim, c = i % obs_dim;
        float v = 0.f;
        if (b0 + e < a.B) {
            const int64_t off = (b0 + e) * a.obs_ld + c;
            v = a.obs_f32 ? io::round(static_cast<const float*>(a.obs)[off]) : io::ld(a.obs, off);
        }
        so[i] = v;
    }
    __syncthreads();
    for (int f = threadIdx.x; f < a.d; f += blockDim.x) {
        float ap[EPB];
        float ao[EPB][NMAX];
#pragma unroll
        for (int e = 0; e < EPB; ++e) {
            ap[e] = 0.f;
#pragma unroll
            for (int j = 0; j < NMAX; ++j) ao[e][j] = 0.f;
        }
        for (int k = 0; k < a.prop_dim; ++k) {
            const float w = io::ld(a.wp, (int64_t)f * a.prop_dim + k);
#pragma unroll
            for (int e = 0; e < EPB; ++e) ap[e] = fmaf(w, so[e * obs_dim + k], ap[e]);
        }
        for (int k = 0; k < a.obj_dim; ++k) {
            const float w = io::ld(a.wo, (int64_t)f * a.obj_dim + k);
#pragma unroll
            for (int e = 0; e < EPB; ++e)
#pragma unroll
                for (int j = 0; j < NMAX; ++j)
                    if (j < nobj) ao[e][j] = fmaf(w, so[e * obs_dim + a.prop_dim + j * a.obj_dim + k], ao[e][j]);
        }
        const float bpv = a.bp ? a.bp[f] : 0.f, bov = a.bo ? a.bo[f] : 0.f;
#pragma unroll
        for (int e = 0; e < EPB; ++e) {
            if (b0 + e >= a.B) break;
            const int64_t base = (b0 + e) * (int64_t)a.T * a.d + f;
            io::st(a.tokens, base, ap[e] + bpv);
#pragma unroll
            for (int j = 0; j < NMAX; ++j) if (j < nobj) io::st(a.tokens, base + (int64_t)(j + 1) * a.d, ao[e][j] + bov);
        }
    }
}

template <typename IO>
int launch(const EmbedArgs& a, hipStream_t st) {
    const int obs_dim = a.prop_dim + (a.T - 1) * a.obj_dim;
    const size_t lds = (size_t)EPB * obs_dim * sizeof(float);
    const unsigned grid = (unsigned)((a.B + EPB - 1) / EPB);
    int threads = ((a.d + 63) / 64) * 64; if (threads > 256) threads = 256;
    if (a.T <= 16) hipLaunchKernelGGL((cfg_embed_kernel<IO, 15>), dim3(grid), dim3(threads), lds, st, a);
    else if (a.T <= 32) hipLaunchKernelGGL((cfg_embed_kernel<IO, 31>), dim3(grid), dim3(threads), lds, st, a);
    else if (a.T <= BSRL_MAX_T) hipLaunchKernelGGL((cfg_embed_kernel<IO, 47>), dim3(grid), dim3(threads), lds, st, a);
    else return BSRL_UNSUPPORTED;
    return BSRL_OK;
}

}  // namespace

extern "C" int bsrl_cfg_embed(const void* obs, int64_t obs_ld, int obs_dtype, const void* wp, const float* bp,
                              const void* wo, const float* bo, void* tokens, int64_t B, int64_t T, int64_t d,
                              int64_t prop_dim, int64_t obj_dim, int dtype, bsrl_stream stream) {
    if (!obs || !wp || !wo || !tokens) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_embed: null pointer");
    if (B < 0 || T < 2 || d <= 0 || prop_dim <= 0 || obj_dim <= 0) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_embed: bad shape");
    if (obs_ld < prop_dim + (T - 1) * obj_dim) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_embed: obs_ld smaller than obs row");
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_embed: bad dtype");
    if (obs_dtype != BSRL_F32 && obs_dtype != dtype) BSRL_FAIL(BSRL_EINVAL, "bsrl_cfg_embed: obs must be F32 or the stream dtype");
    if (B == 0) return BSRL_OK;
    if ((prop_dim + (T - 1) * obj_dim) * 4 * EPB > 60000) return BSRL_UNSUPPORTED;
    EmbedArgs a{obs, obs_ld, obs_dtype == BSRL_F32, wp, bp, wo, bo, tokens, B, (int)T, (int)d, (int)prop_dim, (int)obj_dim};
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc;
    if (dtype == BSRL_F32) rc = launch<F32IO>(a, st);
    else if (dtype == BSRL_F16) rc = launch<F16>(a, st);
    else rc = launch<BF16>(a, st);
    if (rc == BSRL_OK) BSRL_CHECK_LAUNCH("bsrl_cfg_embed");
    return rc;
}
