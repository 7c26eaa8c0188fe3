// Shared device helpers for the gfx950 policy-forward kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/bsrl.h"

typedef uint16_t u16;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define WAVE 64

// ---- host-side error plumbing ------------------------------------------------
void bsrl_set_error(const char* fmt, ...);
#define BSRL_FAIL(code, ...) do { bsrl_set_error(__VA_ARGS__); return (code); } while (0)
#define BSRL_CHECK_LAUNCH(what) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) BSRL_FAIL(BSRL_ELAUNCH, "%s: %s", what, hipGetErrorString(e_)); } while (0)

static inline bool bsrl_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- 16-bit storage types ------------------------------------------------------
// Activations and weights are held as raw 16-bit words; the tag types below give
// the conversions and the MFMA flavour for each format.
struct F16 {
    static __device__ __forceinline__ float to_f(u16 v) { return (float)__builtin_bit_cast(_Float16, v); }
    static __device__ __forceinline__ u16 from_f(float f) { return __builtin_bit_cast(u16, (_Float16)f); }
    // two roundings in one instruction (v_cvt_pk_f16_f32, round to nearest even): a in the low half
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    // D(16x16) += A(16x32) * B(32x16); lane l holds A[l%16][8*(l/16)..+7], B[8*(l/16)..+7][l%16],
    // D[4*(l/16)+i][l%16].
    static __device__ __forceinline__ f32x4 mfma32(s16x8 a, s16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    // K = 16 flavour: lane l holds A[l%16][4*(l/16)..+3], B[4*(l/16)..+3][l%16].
    static __device__ __forceinline__ f32x4 mfma16(s16x4 a, s16x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    }
};
struct BF16 {
    static __device__ __forceinline__ float to_f(u16 v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
    // round to nearest even; gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32)
    static __device__ __forceinline__ u16 from_f(float f) { return __builtin_bit_cast(u16, (__bf16)f); }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {          // v_cvt_pk_bf16_f32
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ f32x4 mfma32(s16x8 a, s16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(s16x4 a, s16x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
    }
};
// fp32 "storage" tag for the kernels that are templated on the I/O type
struct F32IO { };

template <typename DT> __device__ __forceinline__ float io_load(const u16* p) { return DT::to_f(*p); }
template <typename DT> __device__ __forceinline__ void io_store(u16* p, float v) { *p = DT::from_f(v); }

// ---- activations ---------------------------------------------------------------
// max(x, 0) as ONE instruction (v_med3_f32 x, 0, +inf): fmaxf(x, 0) compiles to a canonicalising v_max_f32 x, x plus the
// max itself, and the epilogues that apply it are bound by VALU issue.  Same value for every non-NaN x (-0 gives +0).
__device__ __forceinline__ float relu1(float x) { return __builtin_amdgcn_fmed3f(x, 0.0f, __builtin_inff()); }

__device__ __forceinline__ float gelu_exact(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
template <int ACT> __device__ __forceinline__ float apply_act(float x) {
    if (ACT == BSRL_ACT_RELU) return relu1(x);
    if (ACT == BSRL_ACT_GELU) return gelu_exact(x);
    return x;
}
// GELU(x) = x * Phi(x) with Phi(x) ~= sigmoid(x * (c0 + c1 x^2 + c2 x^4)): 7 full-rate ops + exp2 + rcp.
// Coefficients are a minimax fit of x * sigmoid(.) to the exact-erf GELU on [-9, 9]: max abs error
// 2.5e-5, below half an fp16 ulp of any value >= 0.06, so it is only used where the result is rounded
// to a 16-bit type straight after.  The polynomial argument is clamped to [-9, 9], outside which the
// sigmoid is 0 / 1 to fp32 precision anyway.
__device__ __forceinline__ float gelu_fast(float x) {
    constexpr float L2E = 1.44269504088896340736f;
    constexpr float C0 = -1.59501576f * L2E, C1 = -7.40113019e-02f * L2E, C2 = 7.03035067e-04f * L2E;
    const float xc = __builtin_amdgcn_fmed3f(x, -9.0f, 9.0f);
    const float x2 = xc * xc;
    float q = fmaf(C2, x2, C1);
    q = fmaf(q, x2, C0);
    const float e = __builtin_amdgcn_exp2f(xc * q);          // exp(-u)
    return x * __builtin_amdgcn_rcpf(e + 1.0f);
}
// The same activation in two pieces, for callers that pin VALU work between MFMAs: the head is the
// two ops that depend on nothing but x (clamp, square), the tail is the rest of the chain.
struct Act16Head { float xc, x2; };
template <int ACT> __device__ __forceinline__ Act16Head act16_head(float x) {
    Act16Head h = {x, x};
    if (ACT == BSRL_ACT_GELU) { h.xc = __builtin_amdgcn_fmed3f(x, -9.0f, 9.0f); h.x2 = h.xc * h.xc; }
    return h;
}
template <int ACT> __device__ __forceinline__ float act16_tail(float x, Act16Head h) {
    if (ACT == BSRL_ACT_RELU) return relu1(x);
    if (ACT == BSRL_ACT_GELU) {
        constexpr float L2E = 1.44269504088896340736f;
        constexpr float C0 = -1.59501576f * L2E, C1 = -7.40113019e-02f * L2E, C2 = 7.03035067e-04f * L2E;
        float q = fmaf(C2, h.x2, C1);
        q = fmaf(q, h.x2, C0);
        const float e = __builtin_amdgcn_exp2f(h.xc * q);
        return x * __builtin_amdgcn_rcpf(e + 1.0f);
    }
    return x;
}
// Pins an fp32 value in a register.  Where an activation's last multiply is followed directly by the conversion to
// fp16, the compiler fuses the two into v_fma_mixlo_f16 (ONE rounding); kernels in which a branch or another op sits
// between them round twice.  All linear kernels must produce the same bits for a row (a row's result may not depend
// on which kernel its batch size selects), so the fused form is kept out where the pattern can arise.
__device__ __forceinline__ float keep_f32(float v) { asm("" : "+v"(v)); return v; }

// activation for values about to be rounded to fp16 / bf16
template <int ACT> __device__ __forceinline__ float apply_act16(float x) {
    if (ACT == BSRL_ACT_RELU) return relu1(x);
    if (ACT == BSRL_ACT_GELU) return gelu_fast(x);
    return x;
}

// ---- wave-level reductions -------------------------------------------------------
// gfx950's lane-row exchanges, as plain VALU instructions (no LDS round trip, no lgkmcnt wait behind the weight
// fragment reads).  A wave is four rows of 16 lanes.  v_permlane16_swap_b32 a, b: rows 1 and 3 of a change places
// with rows 0 and 2 of b; v_permlane32_swap_b32 a, b: rows 2..3 of a with rows 0..1 of b.  Written as asm because
// the compiler builtin returns the first result twice in this toolchain; the s_nop is the two wait states the
// instruction needs after a VALU write of either operand (the compiler does not look inside an asm statement).
__device__ __forceinline__ void row_swap16(float& a, float& b) { asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void row_swap32(float& a, float& b) { asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
// The lane-row butterfly (combine with lane ^ 16, then with lane ^ 32) of TWO values at once: on return every lane
// holds the combination of its column over the four rows, for both values, associated (r0 . r1) . (r2 . r3) exactly
// as the two-step shuffle butterfly associates it.  8 VALU ops for the pair.
template <typename OP> __device__ __forceinline__ void rows_reduce2(float& s, float& q, OP op) {
    row_swap16(s, q);                   // s = {s0, q0, s2, q2}, q = {s1, q1, s3, q3} (by row)
    float z = op(s, q), w = z;          // {s0.s1, q0.q1, s2.s3, q2.q3}
    row_swap32(z, w);                   // z = {z0, z1, z0, z1}, w = {z2, z3, z2, z3}
    float t = op(z, w), u = t;          // {S, Q, S, Q}
    row_swap16(t, u);                   // t = {S, S, S, S}, u = {Q, Q, Q, Q}
    s = t; q = u;
}
struct OpAdd { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct OpMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };

// Butterfly over the low `width` lanes of each width-aligned lane group.
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int o = WIDTH / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
template <int WIDTH> __device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int o = WIDTH / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
