// Shared pieces of the full-precision chunk form (wkv6_chunk32_fwd.hip, wkv6_chunk32_bwd.hip): the WKV6
// recurrence over chunks of 32 tokens with every operand in fp32 on v_mfma_f32_16x16x4_f32.
//
// Within a chunk that starts at state S_0, with d_t = -exp(w_t) the log decay of token t and
// c_t = sum_{p<t} d_p (c_0 = 0, m = c_16, c_32 the whole chunk):
//   y_t   = R'_t S_0 + sum_{s<t} A[t][s] v_s + (sum_i r_t u k_t) v_t ,  A[t][s] = sum_i R~_t[i] K~_s[i]
//   S_32  = e^{c_32} o S_0 + K'^T V
//   R'_t = r_t e^{c_t}           K'_s = k_s e^{c_32 - c_{s+1}}       (factors <= 1)
//   R~_t = r_t e^{c_t - m}       K~_s = k_s e^{m - c_{s+1}}          (factors within e^{+-kC32Reach})
// (R~ K~^T needs only t > s: one factor of each such product is <= 1 and the other bounded by the reach.)
// A pair whose decay sums leave that reach inside some chunk is redone by the per-timestep kernels.
//
// Fragment convention of v_mfma_f32_16x16x4_f32 (lane l: n = l & 15, g = l >> 4): A holds row n, k = g;
// B holds k = g, column n; C/D holds column n, rows 4g .. 4g+3.  A sum over 16 indices takes four
// instructions v = 0..3; the index handled by k-slot g of instruction v is 4g + v, so that a C/D tile can
// be fed back as the B operand of a later product without moving it.
#pragma once
#include "wkv6_common.h"

namespace wkv6 {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Four consecutive elements as they sit in memory, converted when they are used: a 16-bit load whose conversion
// stood next to it would make the wave wait for the load where it is issued.
template <typename T> struct Raw4;
template <> struct Raw4<float> {
    f32x4 x;
    __device__ __forceinline__ void load(const float *p) { x = *reinterpret_cast<const f32x4 *>(p); }
    __device__ __forceinline__ float at(int i) const { return x[i]; }
};
template <> struct Raw4<f16_t> {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 x;
    __device__ __forceinline__ void load(const f16_t *p) { x = *reinterpret_cast<const h4 *>(p); }
    __device__ __forceinline__ float at(int i) const { return (float)x[i]; }
};

constexpr int kC32 = 32;            // tokens per chunk
constexpr int kLd = 68;             // floats per row of a [token][channel] LDS tile (64 + 4: 16-byte fragment reads without bank conflicts)
constexpr int kLa = 36;             // floats per row of a [token][token] LDS tile
constexpr float kC32Reach = 40.f;   // largest |sum of log decays| over half a chunk that the scaled operands are formed for

__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
// D += A B over 16 indices: a[v], b[v] are the operands of instruction v
__device__ __forceinline__ f32x4 mfma16(const f32x4 a, const f32x4 b, f32x4 c) {
    c = mfma4(a[0], b[0], c);
    c = mfma4(a[1], b[1], c);
    c = mfma4(a[2], b[2], c);
    c = mfma4(a[3], b[3], c);
    return c;
}

// x of the lane `kCtrl` away inside the row of 16 (DPP row_shr:n = 0x110 + n, row_shl:n = 0x100 + n); 1 where the row ends
template <int kCtrl> __device__ __forceinline__ float row_take(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0x3f800000, __float_as_int(x), kCtrl, 0xF, 0xF, false));
}
// running products over the 16 lanes of a row: lane n gets x_0 .. x_n (up) or x_n .. x_15 (down).  One DPP
// multiply per step (a lane without a source keeps its value); the wait states a DPP read of a freshly written
// register needs are spelled out, the compiler does not look inside.
__device__ __forceinline__ float row_product_up(float x) {
    asm("s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf" : "+v"(x));
    return x;
}
__device__ __forceinline__ float row_product_down(float x) {
    asm("s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shl:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shl:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_mul_f32_dpp %0, %0, %0 row_shl:8 row_mask:0xf bank_mask:0xf" : "+v"(x));
    return x;
}
// x of the same lane-in-row in each of the wave's four rows (lanes n, 16 + n, 32 + n, 48 + n), in every lane
__device__ __forceinline__ void rows4(float x, float (&o)[4]) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 s = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);   // (even row, odd row) of the lane's half
    const u32x2 a = __builtin_amdgcn_permlane32_swap(s[0], s[0], false, false);                               // (lower half, upper half)
    const u32x2 b = __builtin_amdgcn_permlane32_swap(s[1], s[1], false, false);
    o[0] = __uint_as_float(a[0]); o[1] = __uint_as_float(b[0]); o[2] = __uint_as_float(a[1]); o[3] = __uint_as_float(b[1]);
}
// sum over the four rows of the wave (lanes l, l ^ 16, l ^ 32, l ^ 48), in every lane
__device__ __forceinline__ float sum_rows4(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 s = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(s[0]) + __uint_as_float(s[1]);
    s = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}
// sum over the 16 lanes of a row, in every lane of it
__device__ __forceinline__ float row_sum16(float x) {
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));   // row_half_mirror
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x140, 0xF, 0xF, true));   // row_mirror
    return x;
}

// A loading wave's share of a chunk: lane (t16 = l & 15, cq = l >> 4) of loading wave p holds channels
// 16p + 4cq .. +3 of tokens t16 (x = 0) and 16 + t16 (x = 1).  The scale factors are running products of
// the per-token decays e^{d_t} (and of their inverses, towards the middle of the chunk) over the 16
// lanes of a row: every exponential sees one token's small argument, as in the per-timestep kernels.
struct C32Scale {
    float rp[2][4];     // e^{c_t}              R' = r rp
    float kp[2][4];     // e^{c_32 - c_{t+1}}   K' = k kp
    float rm[2][4];     // e^{c_t - m}          R~ = r rm
    float km[2][4];     // e^{m - c_{t+1}}      K~ = k km
    float all[4];       // e^{c_32}
    float mid[4];       // e^{m}
    float rest[4];      // e^{c_32 - m}
    float inv0[4];      // e^{-m}
    float inv1[4];      // e^{m - c_32}
    bool wild;          // a half-chunk product outside the reach
};
// raw: the w values (ignored for rows that are not valid, whose decay is 1); d: the log decays -exp(w).
// Channels kFrom .. kTo-1 of the lane's four (o.wild accumulates).
template <int kFrom, int kTo>
__device__ __forceinline__ void c32_scale(const float (&raw)[2][4], const bool (&valid)[2], C32Scale &o, float (&d)[2][4]) {
    const float reach = 4.2e-18f;   // e^{-kC32Reach}
#pragma unroll
    for (int e = kFrom; e < kTo; ++e) {
        d[0][e] = valid[0] ? -fast_exp(raw[0][e]) : 0.f;
        d[1][e] = valid[1] ? -fast_exp(raw[1][e]) : 0.f;
        const float w0 = fast_exp(d[0][e]), w1 = fast_exp(d[1][e]);
        const float up0 = row_product_up(w0), up1 = row_product_up(w1);
        const float dn0 = row_product_down(w0), dn1 = row_product_down(w1);
        // the way back to the chunk's middle: the reciprocal of the product from there (1 ulp, as good as a product
        // of sixteen rounded factors; outside the reach, where it overflows, the pair is redone anyway)
        const float to_mid0 = __builtin_amdgcn_rcpf(dn0), to_mid1 = __builtin_amdgcn_rcpf(up1);
        const float before0 = row_take<0x111>(up0), before1 = row_take<0x111>(up1);   // products of the tokens before this one
        const float after0 = row_take<0x101>(dn0), after1 = row_take<0x101>(dn1);     // ... behind this one
        const float all0 = up0 * after0, all1 = up1 * after1;                         // the whole row (each lane's own rounding of it)
        o.rp[0][e] = before0;        o.rp[1][e] = all0 * before1;
        o.kp[0][e] = after0 * all1;  o.kp[1][e] = after1;
        o.rm[0][e] = to_mid0;        o.rm[1][e] = before1;
        o.km[0][e] = after0;         o.km[1][e] = to_mid1;
        o.all[e] = all0 * all1;
        o.mid[e] = all0;
        o.rest[e] = all1;
        o.inv0[e] = __builtin_amdgcn_rcpf(all0);
        o.inv1[e] = __builtin_amdgcn_rcpf(all1);
        o.wild |= !(all0 >= reach) || !(all1 >= reach);   // (NaN counts as outside)
    }
}

}  // namespace wkv6
