// Shared device helpers for the WKV6 kernels (gfx950 only, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wkv6 {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

constexpr int kN = 64;  // head size the kernels are built for

__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }
// decay d = exp(-exp(w)); w = -1e9 gives exactly 1, w >= ~5 gives exactly 0, never NaN for finite w.
__device__ __forceinline__ float decay_from_raw(float w) { return __expf(-__expf(w)); }

__device__ __forceinline__ float bf16_bits_to_float(uint32_t hi16) { return __uint_as_float(hi16 << 16); }
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (x >> 16) | 0x40u;  // NaN stays NaN
    return (x + 0x7fffu + ((x >> 16) & 1u)) >> 16;                   // round to nearest even
}
// two fp32 -> packed bf16x2, round to nearest even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const f32x2_t t = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(t, bf16x2_t));
}

// Eight consecutive elements as they sit in memory; converted to fp32 only when consumed, so a
// prefetch held across a compute phase costs 4 VGPRs for 16-bit types.
template <typename T> struct Raw8;
template <> struct Raw8<float> {
    // (one native vector: as a struct of two of the runtime's float4 the eight values are kept in scratch memory, and a
    // prefetch then waits for its loads at once to store them there)
    typedef float v4 __attribute__((ext_vector_type(4)));
    typedef float v8 __attribute__((ext_vector_type(8)));
    v8 a;
    __device__ __forceinline__ void load(const float *p) {
        const v4 lo = *reinterpret_cast<const v4 *>(p), hi = *reinterpret_cast<const v4 *>(p + 4);
        a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    __device__ __forceinline__ void zero() { a = (v8)(0.f); }
    __device__ __forceinline__ void to_float(float (&o)[8]) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = a[i];
    }
};
template <> struct Raw8<bf16_t> {
    uint4 a;
    __device__ __forceinline__ void load(const bf16_t *p) { a = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ void zero() { a = make_uint4(0, 0, 0, 0); }
    __device__ __forceinline__ void to_float(float (&o)[8]) const {
        o[0] = __uint_as_float(a.x << 16); o[1] = __uint_as_float(a.x & 0xffff0000u);
        o[2] = __uint_as_float(a.y << 16); o[3] = __uint_as_float(a.y & 0xffff0000u);
        o[4] = __uint_as_float(a.z << 16); o[5] = __uint_as_float(a.z & 0xffff0000u);
        o[6] = __uint_as_float(a.w << 16); o[7] = __uint_as_float(a.w & 0xffff0000u);
    }
};
template <> struct Raw8<f16_t> {
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    h8 a;
    __device__ __forceinline__ void load(const f16_t *p) { a = *reinterpret_cast<const h8 *>(p); }
    __device__ __forceinline__ void zero() { a = (h8)(0); }
    __device__ __forceinline__ void to_float(float (&o)[8]) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (float)a[i];
    }
};

// Store n (4 or 8) consecutive fp32 values as the output type, one vector store.
__device__ __forceinline__ void store4(float *p, float a, float b, float c, float d) {
    *reinterpret_cast<float4 *>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16_t *p, float a, float b, float c, float d) {
    *reinterpret_cast<uint2 *>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}
__device__ __forceinline__ void store1(float *p, float a) { *p = a; }
__device__ __forceinline__ void store1(bf16_t *p, float a) {
    *reinterpret_cast<uint16_t *>(p) = (uint16_t)pack_bf16x2(a, 0.f);
}
// four consecutive elements as fp32, one vector load
__device__ __forceinline__ void load4(const float *p, float (&o)[4]) {
    const float4 x = *reinterpret_cast<const float4 *>(p);
    o[0] = x.x; o[1] = x.y; o[2] = x.z; o[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t *p, float (&o)[4]) {
    const uint2 x = *reinterpret_cast<const uint2 *>(p);
    o[0] = __uint_as_float(x.x << 16); o[1] = __uint_as_float(x.x & 0xffff0000u);
    o[2] = __uint_as_float(x.y << 16); o[3] = __uint_as_float(x.y & 0xffff0000u);
}
__device__ __forceinline__ void load4(const f16_t *p, float (&o)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 x = *reinterpret_cast<const h4 *>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (float)x[i];
}
__device__ __forceinline__ float load1(const float *p) { return *p; }
__device__ __forceinline__ float load1(const bf16_t *p) {
    return bf16_bits_to_float(*reinterpret_cast<const uint16_t *>(p));
}
__device__ __forceinline__ float load1(const f16_t *p) { return (float)*p; }

}  // namespace wkv6
