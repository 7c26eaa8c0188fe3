// NotePolicy front end: one pass over the (B, 630) observation that writes every encoder
// input of the forward and the additive key bias.
//
// Replaces, for the reference's forward preamble (python/policy.py:1199-1260): the one-time
// rounding of the obs to the stream dtype (:1199-1209), the two lane gathers and the entity
// views of `_split` (:1099-1105), the 22 note-geometry lanes of `_note_geo` (:329-404,
// fp32 arithmetic on the rounded lanes, rounded once on store), the hand / side one-hot
// concatenations (:1231-1246) and the key-bias build (:1257-1260).
//
// A workgroup owns EPB envs.  Their obs rows are read once (coalesced), rounded to the stream
// dtype and parked in LDS as fp32; every output is then produced from LDS and stored with
// consecutive threads on consecutive elements.  HBM traffic per env is the algorithmic
// minimum: 630 elements in, 98 + 29 + 68 + 24 * (18 | 40) + 29 elements out.
#include "bsrl_common.h"

namespace {

constexpr int EPB = 8;
constexpr int OBS_DIM = 630, N_SLOTS = 24, NOTE_FEAT = 18, GEO_FEAT = 22;
constexpr int OFF_NOTES = 102, OFF_MASK = OFF_NOTES + N_SLOTS * NOTE_FEAT, OBS_HEAD_Z = 99;
constexpr int SABER_FEAT = 47, TORSO_FEAT = 29, LEG_FEAT = 32, N_LEAD = 5, T_TOK = N_LEAD + N_SLOTS;
// lanes inside a saber token and the env's obs normalisers (python/policy.py:319-326)
constexpr int S_WPOS = 15, S_WVEL = 18, S_BLADE = 21, S_TIPV = 44;
constexpr float X_NORM = 1.0f, Y_NORM = 0.75f, Z_SCALE = 8.0f, V_NORM = 6.0f, HANDLE_LEN = 0.16f;
constexpr float MASK_BIAS = 16384.0f;
constexpr int PITCH = 64;                      // row pitch of the padded encoder inputs

struct FrontArgs {
    const void* obs; int64_t obs_ld; int obs_dtype;
    const int32_t* saber_idx;      // 2 * 47 obs lanes: left hand, right hand
    const int32_t* body_idx;       // 29 torso + 32 left-leg + 32 right-leg obs lanes
    int note_geo, flux; float z_asinh;
    void* saber_in; void* torso_in; void* leg_in; void* note_in; void* key_bias;
    int64_t B;
};

template <typename IO> struct FIO;
template <> struct FIO<F32IO> {
    static __device__ __forceinline__ float round(float v) { return v; }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
};
template <typename DT> struct FIO16 {
    static __device__ __forceinline__ float round(float v) { return DT::to_f(DT::from_f(v)); }
    static __device__ __forceinline__ void st(void* p, int64_t i, float v) { static_cast<u16*>(p)[i] = DT::from_f(v); }
};
template <> struct FIO<F16> : FIO16<F16> {};
template <> struct FIO<BF16> : FIO16<BF16> {};

__device__ __forceinline__ float load_obs(const void* p, int64_t i, int dtype) {
    if (dtype == BSRL_F32) return static_cast<const float*>(p)[i];
    if (dtype == BSRL_F16) return F16::to_f(static_cast<const u16*>(p)[i]);
    return BF16::to_f(static_cast<const u16*>(p)[i]);
}

struct V3 { float x, y, z; };
__device__ __forceinline__ float dot3(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ __forceinline__ float norm3(V3 a) { return sqrtf(dot3(a, a)); }

template <typename IO, bool PAD>
__global__ __launch_bounds__(256) void note_frontend_kernel(FrontArgs a) {
    typedef FIO<IO> io;
    __shared__ float so[EPB][OBS_DIM + 2];
    __shared__ float sgeo[EPB][N_SLOTS][GEO_FEAT];
    __shared__ int s_sab[2 * SABER_FEAT], s_body[TORSO_FEAT + 2 * LEG_FEAT];
    const int tid = threadIdx.x;
    const int64_t b0 = (int64_t)blockIdx.x * EPB;
    const int nenv = (int)((a.B - b0) < EPB ? (a.B - b0) : EPB);

    for (int i = tid; i < 2 * SABER_FEAT; i += 256) s_sab[i] = a.saber_idx[i];
    for (int i = tid; i < TORSO_FEAT + 2 * LEG_FEAT; i += 256) s_body[i] = a.body_idx[i];
    // dense fp32 rows (the rollout's obs buffer): the workgroup's 8 rows are one contiguous, 16-byte aligned block -
    // every 16-byte load of a thread is issued before the first LDS write.  The general loop below pays one memory
    // round trip per element (the dtype switch keeps its loads apart): 20 of them per thread.
    if (a.obs_dtype == BSRL_F32 && a.obs_ld == OBS_DIM && nenv == EPB && (reinterpret_cast<uintptr_t>(a.obs) & 15) == 0) {
        constexpr int NP = EPB * OBS_DIM / 4, NITF = (NP + 255) / 256;
        static_assert(EPB * OBS_DIM % 4 == 0, "a workgroup's obs block is a whole number of 16-byte pieces");
        const float4* src = reinterpret_cast<const float4*>(static_cast<const float*>(a.obs) + b0 * OBS_DIM);
        float4 v[NITF];
#pragma unroll
        for (int it = 0; it < NITF; ++it) {
            const int p = it * 256 + tid;
            v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p < NP) v[it] = src[p];
        }
#pragma unroll
        for (int it = 0; it < NITF; ++it) {
            const int p = it * 256 + tid;
            if (p < NP) {
                const float f[4] = {v[it].x, v[it].y, v[it].z, v[it].w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int i = 4 * p + k, e = i / OBS_DIM, c = i - e * OBS_DIM;
                    so[e][c] = io::round(f[k]);
                }
            }
        }
    } else {
        for (int i = tid; i < nenv * OBS_DIM; i += 256) {
            const int e = i / OBS_DIM, c = i - e * OBS_DIM;
            so[e][c] = io::round(load_obs(a.obs, (b0 + e) * a.obs_ld + c, a.obs_dtype));
        }
    }
    __syncthreads();

    // ---- note geometry: one thread per (env, slot) ----
    if (a.note_geo) {
        for (int p = tid; p < nenv * N_SLOTS; p += 256) {
            const int e = p / N_SLOTS, s = p - e * N_SLOTS;
            const float* n = &so[e][OFF_NOTES + s * NOTE_FEAT];
            float* out = sgeo[e][s];
            const float z_m = sinhf(n[2]) * a.z_asinh;
            float tx = n[0], ty = n[1];
            if (a.flux && n[9] > 0.5f) { tx = n[12]; ty = n[13]; }
            const V3 npos = {tx * X_NORM, ty * Y_NORM, z_m};
            const V3 cutd = {n[6], n[7], 0.f};
            const float not_wall = 1.0f - n[14];
            const float speed = fmaxf(-n[3] * Z_SCALE, 1e-3f);
            const float tpl = fminf(fmaxf((z_m - so[e][OBS_HEAD_Z] * X_NORM) / speed, -0.5f), 3.0f) / 3.0f;
#pragma unroll
            for (int hand = 0; hand < 2; ++hand) {
                // the saber token's lanes, read through the gather table
                auto w = [&](int lane) { return so[e][s_sab[hand * SABER_FEAT + lane]]; };
                const V3 wpos = {w(S_WPOS) * X_NORM, w(S_WPOS + 1) * Y_NORM, w(S_WPOS + 2)};
                const V3 dpm = {npos.x - wpos.x, npos.y - wpos.y, npos.z - wpos.z};
                const V3 dp = {dpm.x * 0.5f, dpm.y * 0.5f, dpm.z * 0.5f};
                const V3 v = {w(S_WVEL) * V_NORM, w(S_WVEL + 1) * V_NORM, w(S_WVEL + 2) * V_NORM};
                const float vs = 1.0f / (norm3(v) + 0.05f);
                const V3 vhat = {v.x * vs, v.y * vs, v.z * vs};
                const V3 b = {w(S_BLADE), w(S_BLADE + 1), w(S_BLADE + 2)};
                float* base = out + hand * 7;
                base[0] = dp.x; base[1] = dp.y; base[2] = asinhf(dp.z * 0.25f);
                base[3] = asinhf(norm3(dp) * 0.25f);
                base[4] = tpl;
                base[5] = dot3(vhat, cutd) * not_wall;
                base[6] = dot3(b, cutd) * not_wall;
                const float ab = dot3(dpm, b);
                const V3 vt = {w(S_TIPV), w(S_TIPV + 1), w(S_TIPV + 2)};
                const V3 vtn = {vt.x * V_NORM, vt.y * V_NORM, vt.z * V_NORM};
                const V3 pn = {b.y * vtn.z - b.z * vtn.y, b.z * vtn.x - b.x * vtn.z, b.x * vtn.y - b.y * vtn.x};
                const float ps = 1.0f / (norm3(pn) + 0.05f);
                const V3 nhat = {pn.x * ps, pn.y * ps, pn.z * ps};
                const V3 perp = {dpm.x - ab * b.x, dpm.y - ab * b.y, dpm.z - ab * b.z};
                float* blade = out + 14 + hand * 4;
                blade[0] = asinhf((ab - HANDLE_LEN) * 0.5f);
                blade[1] = asinhf(norm3(perp) * 0.5f);
                blade[2] = asinhf(dot3(dpm, nhat) * 0.5f);
                blade[3] = dot3(vt, cutd) * not_wall;
            }
        }
        __syncthreads();
    }

    // ---- stores: each output tensor is contiguous over the workgroup's envs ----
    // PAD: every encoder-input row is PITCH elements long, zero past its natural width, so the first encoder
    // Linear runs as a K = PITCH GEMM on the vector kernels (zeros add nothing to the fp32 accumulators)
    constexpr int SAB_W = SABER_FEAT + 2, LEG_W = LEG_FEAT + 2;
    constexpr int SAB_P = PAD ? PITCH : SAB_W, TOR_P = PAD ? PITCH : TORSO_FEAT, LEG_P = PAD ? PITCH : LEG_W;
    for (int i = tid; i < nenv * 2 * SAB_P; i += 256) {            // (B, 2, 49): 47 lanes + hand one-hot
        const int e = i / (2 * SAB_P), r = i - e * 2 * SAB_P, hand = r / SAB_P, c = r - hand * SAB_P;
        const float v = c < SABER_FEAT ? so[e][s_sab[hand * SABER_FEAT + c]]
                                       : (c < SAB_W && c - SABER_FEAT == hand ? 1.f : 0.f);
        io::st(a.saber_in, b0 * 2 * SAB_P + i, v);
    }
    for (int i = tid; i < nenv * TOR_P; i += 256) {                // (B, 29)
        const int e = i / TOR_P, c = i - e * TOR_P;
        io::st(a.torso_in, b0 * TOR_P + i, c < TORSO_FEAT ? so[e][s_body[c]] : 0.f);
    }
    for (int i = tid; i < nenv * 2 * LEG_P; i += 256) {            // (B, 2, 34): 32 lanes + side one-hot
        const int e = i / (2 * LEG_P), r = i - e * 2 * LEG_P, side = r / LEG_P, c = r - side * LEG_P;
        const float v = c < LEG_FEAT ? so[e][s_body[TORSO_FEAT + side * LEG_FEAT + c]]
                                     : (c < LEG_W && c - LEG_FEAT == side ? 1.f : 0.f);
        io::st(a.leg_in, b0 * 2 * LEG_P + i, v);
    }
    const int NW = NOTE_FEAT + (a.note_geo ? GEO_FEAT : 0);
    const int NP_ = PAD ? PITCH : NW;
    for (int i = tid; i < nenv * N_SLOTS * NP_; i += 256) {        // (B, 24, 18 | 40)
        const int p = i / NP_, c = i - p * NP_, e = p / N_SLOTS, s = p - e * N_SLOTS;
        const float v = c < NOTE_FEAT ? so[e][OFF_NOTES + s * NOTE_FEAT + c] : (c < NW ? sgeo[e][s][c - NOTE_FEAT] : 0.f);
        io::st(a.note_in, b0 * N_SLOTS * NP_ + i, v);
    }
    for (int i = tid; i < nenv * T_TOK; i += 256) {                // (B, 29): lead tokens always attendable
        const int e = i / T_TOK, t = i - e * T_TOK;
        const float v = t < N_LEAD ? 0.f : (so[e][OFF_MASK + t - N_LEAD] - 1.0f) * MASK_BIAS;
        io::st(a.key_bias, b0 * T_TOK + i, v);
    }
}

}  // namespace

namespace {

int frontend_launch(const char* who, bool pad, const void* obs, int64_t obs_ld, int obs_dtype,
                    const int32_t* saber_idx, const int32_t* body_idx, int note_geo, int flux, float z_asinh,
                    void* saber_in, void* torso_in, void* leg_in, void* note_in, void* key_bias,
                    int64_t B, int dtype, bsrl_stream stream) {
    if (!obs || !saber_idx || !body_idx || !saber_in || !torso_in || !leg_in || !note_in || !key_bias)
        BSRL_FAIL(BSRL_EINVAL, "%s: null pointer", who);
    if (B < 0 || obs_ld < OBS_DIM) BSRL_FAIL(BSRL_EINVAL, "%s: B < 0 or obs_ld < %d", who, OBS_DIM);
    if (dtype != BSRL_F32 && dtype != BSRL_F16 && dtype != BSRL_BF16) BSRL_FAIL(BSRL_EINVAL, "%s: bad dtype %d", who, dtype);
    if (obs_dtype != BSRL_F32 && obs_dtype != dtype)
        BSRL_FAIL(BSRL_EINVAL, "%s: obs must be fp32 or already in the stream dtype", who);
    if (!(z_asinh > 0.f)) BSRL_FAIL(BSRL_EINVAL, "%s: z_asinh must be > 0", who);
    if (B == 0) return BSRL_OK;
    FrontArgs a{obs, obs_ld, obs_dtype, saber_idx, body_idx, note_geo != 0, flux != 0, z_asinh,
                saber_in, torso_in, leg_in, note_in, key_bias, B};
    const dim3 grid((unsigned)((B + EPB - 1) / EPB)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define BSRL_FRONT(IO)                                                                   \
    do {                                                                                 \
        if (pad) hipLaunchKernelGGL((note_frontend_kernel<IO, true>), grid, block, 0, st, a);  \
        else hipLaunchKernelGGL((note_frontend_kernel<IO, false>), grid, block, 0, st, a);     \
    } while (0)
    if (dtype == BSRL_F32) BSRL_FRONT(F32IO);
    else if (dtype == BSRL_F16) BSRL_FRONT(F16);
    else BSRL_FRONT(BF16);
#undef BSRL_FRONT
    BSRL_CHECK_LAUNCH(who);
    return BSRL_OK;
}

}  // namespace

extern "C" int bsrl_note_frontend(const void* obs, int64_t obs_ld, int obs_dtype,
                                  const int32_t* saber_idx, const int32_t* body_idx,
                                  int note_geo, int flux, float z_asinh,
                                  void* saber_in, void* torso_in, void* leg_in, void* note_in, void* key_bias,
                                  int64_t B, int dtype, bsrl_stream stream) {
    return frontend_launch("bsrl_note_frontend", false, obs, obs_ld, obs_dtype, saber_idx, body_idx, note_geo, flux,
                           z_asinh, saber_in, torso_in, leg_in, note_in, key_bias, B, dtype, stream);
}

extern "C" int bsrl_note_frontend_padded(const void* obs, int64_t obs_ld, int obs_dtype,
                                         const int32_t* saber_idx, const int32_t* body_idx,
                                         int note_geo, int flux, float z_asinh,
                                         void* saber_in, void* torso_in, void* leg_in, void* note_in, void* key_bias,
                                         int64_t B, int dtype, bsrl_stream stream) {
    return frontend_launch("bsrl_note_frontend_padded", true, obs, obs_ld, obs_dtype, saber_idx, body_idx, note_geo,
                           flux, z_asinh, saber_in, torso_in, leg_in, note_in, key_bias, B, dtype, stream);
}
