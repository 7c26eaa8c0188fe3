// Row-chunk loads / stores of the LayerNorm kernels: a lane moves 16 bytes (4 fp32 or 8 16-bit
// elements) at a time and works on them in fp32.
#pragma once
#include "bsrl_common.h"

namespace {

template <typename IO> struct LnIO;
template <> struct LnIO<F32IO> {
    static constexpr int VEC = 4;
    typedef float elem;
    typedef float4 raw;
    static __device__ __forceinline__ raw load_raw(const void* p, int64_t off) {
        return *reinterpret_cast<const float4*>(static_cast<const float*>(p) + off);
    }
    static __device__ __forceinline__ void cvt(raw t, float* v) { v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
    static __device__ __forceinline__ void load(const void* p, int64_t off, float* v) { cvt(load_raw(p, off), v); }
    static __device__ __forceinline__ void store(void* p, int64_t off, const float* v) {
        *reinterpret_cast<float4*>(static_cast<float*>(p) + off) = make_float4(v[0], v[1], v[2], v[3]);
    }
    static __device__ __forceinline__ float round(float v) { return v; }
};
template <typename DT> struct LnIO16 {
    static constexpr int VEC = 8;
    typedef uint4 raw;
    static __device__ __forceinline__ raw load_raw(const void* p, int64_t off) {
        return *reinterpret_cast<const uint4*>(static_cast<const u16*>(p) + off);
    }
    static __device__ __forceinline__ void cvt(raw t, float* v) {
        uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[2 * i] = DT::to_f((u16)(w[i] & 0xffff)); v[2 * i + 1] = DT::to_f((u16)(w[i] >> 16)); }
    }
    static __device__ __forceinline__ void load(const void* p, int64_t off, float* v) { cvt(load_raw(p, off), v); }
    static __device__ __forceinline__ void store(void* p, int64_t off, const float* v) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = (uint32_t)DT::from_f(v[2 * i]) | ((uint32_t)DT::from_f(v[2 * i + 1]) << 16);
        *reinterpret_cast<uint4*>(static_cast<u16*>(p) + off) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    static __device__ __forceinline__ float round(float v) { return DT::to_f(DT::from_f(v)); }
};
template <> struct LnIO<F16> : LnIO16<F16> {};
template <> struct LnIO<BF16> : LnIO16<BF16> {};

}  // namespace
