// MFMA fragment helpers shared by the chunked WKV6 kernels (gfx950, wave64).
#pragma once
#include "wkv6_common.h"

namespace wkv6 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int LDA = 68;  // row pitch (elements) of [token][channel] operand arrays: 136 B, conflict-free 8-byte fragment reads
constexpr float kWildLimit = 64.f;
constexpr float kLog2e = 1.4426950408889634f;
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }   // v_exp_f32

__device__ __forceinline__ bf16x8 make_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const u32x4 t = {a, b, c, d};
    return __builtin_bit_cast(bf16x8, t);
}
__device__ __forceinline__ s16x4 make_s16x4(uint32_t a, uint32_t b) {
    const u32x2 t = {a, b};
    return __builtin_bit_cast(s16x4, t);
}
__device__ __forceinline__ f32x4 mfma32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(s16x4 a, s16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}
// Two software-inserted delays around the MFMAs.  Both pass the accumulators through an asm
// statement, so neither the MFMAs that write them nor the code that reads them can move across.
//
// chain_gap(acc): 8 idle issue slots between two MFMAs of DIFFERENT shape (16x16x16 and 16x16x32)
// that are chained through the same accumulator.  hipcc 7.2 schedules such a pair 0-3 slots apart,
// and on gfx950 the second MFMA then reads a stale SrcC: the products came out wrong whenever the
// scheduler happened to place the pair that close and right when it left 5 or more slots.
// Same-shape accumulation chains are not affected.
//
// settle(acc...): 16 idle slots before VALU code (masks, scaling, bf16 conversion, stores) reads
// MFMA results; belt and braces on top of the wait states the compiler inserts itself.
#define WKV6_SETTLE_ASM "s_nop 15"
__device__ __forceinline__ void chain_gap(f32x4 &a) { asm volatile("s_nop 7" : "+v"(a)); }
__device__ __forceinline__ void settle(f32x4 &a) { asm volatile(WKV6_SETTLE_ASM : "+v"(a)); }
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b) { asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b, f32x4 (&g1)[4]) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b), "+v"(g1[0]), "+v"(g1[1]), "+v"(g1[2]), "+v"(g1[3]));
}
__device__ __forceinline__ void settle(f32x4 &a, f32x4 (&g1)[4]) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(g1[0]), "+v"(g1[1]), "+v"(g1[2]), "+v"(g1[3]));
}
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b, f32x4 &c) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b), "+v"(c));
}
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b, f32x4 &c, f32x4 &d) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b, f32x4 &c, f32x4 &d, f32x4 &e) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e));
}
__device__ __forceinline__ void settle(f32x4 &a, f32x4 &b, f32x4 &c, f32x4 (&g1)[4], f32x4 (&g2)[4]) {
    asm volatile(WKV6_SETTLE_ASM : "+v"(a), "+v"(b), "+v"(c), "+v"(g1[0]), "+v"(g1[1]), "+v"(g1[2]), "+v"(g1[3]),
                 "+v"(g2[0]), "+v"(g2[1]), "+v"(g2[2]), "+v"(g2[3]));
}
__device__ __forceinline__ float xor1(float x) {   // value of the neighbouring lane (lane ^ 1)
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));
}

// Sum over the four 16-lane rows of the wave (lanes l, l^16, l^32, l^48), result in every lane,
// with the gfx950 row-swap instructions instead of LDS permutes.
__device__ __forceinline__ float sum_rows(float x) {
    const uint32_t xi = __float_as_uint(x);
    const u32x2 a = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);   // rows (0,0,2,2) and (1,1,3,3)
    const uint32_t si = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const u32x2 b = __builtin_amdgcn_permlane32_swap(si, si, false, false);   // rows (0,1,0,1) and (2,3,2,3)
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
// Exclusive prefix over the four rows: row g receives the sum of x over rows 0..g-1.
__device__ __forceinline__ float prefix_rows(float x, int g) {
    const uint32_t xi = __float_as_uint(x);
    const u32x2 a = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);   // a[0] = rows (0,0,2,2), a[1] = rows (1,1,3,3)
    const float below = __uint_as_float(a[0]);                                 // in odd rows: the row just below
    const uint32_t si = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const u32x2 b = __builtin_amdgcn_permlane32_swap(si, si, false, false);   // b[0] = rows 0+1 everywhere
    return ((g & 1) ? below : 0.f) + ((g & 2) ? __uint_as_float(b[0]) : 0.f);
}

// 16-bit load at a uniform base + 32-bit per-lane byte offset (lets the compiler use the
// scalar-base addressing form instead of 64-bit per-lane address arithmetic)
__device__ __forceinline__ uint32_t ld16(const void *base, uint32_t byteoff) {
    return *reinterpret_cast<const uint16_t *>(reinterpret_cast<const char *>(base) + byteoff);
}

// the low / the high bf16 of a packed pair
__device__ __forceinline__ void st16_lo(void *base, uint32_t byteoff, uint32_t pair) {
    *reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(base) + byteoff) = (uint16_t)pair;
}
__device__ __forceinline__ void st16_hi(void *base, uint32_t byteoff, uint32_t pair) {
    *reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(base) + byteoff) = (uint16_t)(pair >> 16);
}
__device__ __forceinline__ void st16(void *base, uint32_t byteoff, float x) {
    *reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(base) + byteoff) = (uint16_t)pack_bf16x2(x, 0.f);
}

// A/B fragment of a [token][channel] array for one 16x16x32 MFMA covering channels [32h, 32h+32).
// Lane group g = lane/16 takes the k-slots {32h+4g+e, 32h+16+4g+e : e<4}: the same channels its
// accumulator registers hold when a 64x16 fp32 tile stack (rows 16m+4g+r) is reused as an operand.
__device__ __forceinline__ bf16x8 frag_tc(const uint16_t (*a)[LDA], int row, int h, int g) {
    const uint2 lo = *reinterpret_cast<const uint2 *>(&a[row][32 * h + 4 * g]);
    const uint2 hi = *reinterpret_cast<const uint2 *>(&a[row][32 * h + 16 + 4 * g]);
    return make_bf16x8(lo.x, lo.y, hi.x, hi.y);
}
// A/B fragment of a [channel][token] array for one 16x16x16 MFMA: 4 consecutive tokens.
template <int LD>
__device__ __forceinline__ s16x4 frag_ct(const uint16_t (*a)[LD], int ch, int tok) {
    const uint2 x = *reinterpret_cast<const uint2 *>(&a[ch][tok]);
    return make_s16x4(x.x, x.y);
}
// two accumulator tiles (rows 16m+4g+r and 16(m+1)+4g+r) as the bf16 operand of a 16x16x32 MFMA
__device__ __forceinline__ bf16x8 acc_as_operand(const f32x4 &a, const f32x4 &b) {
    return make_bf16x8(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(b[0], b[1]), pack_bf16x2(b[2], b[3]));
}

// sum over the 64 lanes of 16 per-lane values; lane l receives the total of value (l>>2)&15.
// The two folds across the 16-lane rows use the row-swap instructions (one swap hands both
// partners what they need), the folds inside a row DPP / the swizzle crossbar.
__device__ __forceinline__ float add_swapped32(float a, float b) {   // rows 0,1: a folded over lane^32; rows 2,3: b
    const u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float add_swapped16(float a, float b) {   // rows 0,2: a folded over lane^16; rows 1,3: b
    const u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float transpose_reduce16(const float (&p)[16], int lane) {
    float x8[8], x4[4], x2[2];
#pragma unroll
    for (int a = 0; a < 8; ++a) x8[a] = add_swapped32(p[a], p[a + 8]);      // value a | a+8 by wave half
#pragma unroll
    for (int a = 0; a < 4; ++a) x4[a] = add_swapped16(x8[a], x8[a + 4]);    // row rho holds value a + 4 rho
    const bool b3 = lane & 8, b2 = lane & 4;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const float keep = b3 ? x4[a + 2] : x4[a], give = b3 ? x4[a] : x4[a + 2];
        x2[a] = keep + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(give), 0x128, 0xF, 0xF, true));   // row_ror:8 = lane^8
    }
    const float keep = b2 ? x2[1] : x2[0], give = b2 ? x2[0] : x2[1];
    float x = keep + __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(give), 0x101F));   // lane^4
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));       // lane^2
    x += xor1(x);
    return x;
}


// Writes row-major [token][channel] bf16 with 4-byte stores: lanes 2c and 2c+1 swap one value so
// that the even lane stores (x[c], x[c+1]) of an even token row and the odd lane those of the
// next row.
__device__ __forceinline__ void store_rows_paired(uint16_t (*a)[LDA], int row0, int lane, const float (&x)[16]) {
    const bool odd = lane & 1;
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        const float got = xor1(odd ? x[e] : x[e + 1]);
        const uint32_t pk = odd ? pack_bf16x2(got, x[e + 1]) : pack_bf16x2(x[e], got);
        *reinterpret_cast<uint32_t *>(&a[row0 + e + (odd ? 1 : 0)][lane & ~1]) = pk;
    }
}

// fragment of a global (B,T,C) bf16 tensor row (uniform base + 32-bit byte offset of the row) for a
// 16x16x32 MFMA, same k-slot order as frag_tc
__device__ __forceinline__ bf16x8 frag_global(const void *base, uint32_t rowbyte, int h, int g) {
    const char *b = reinterpret_cast<const char *>(base);
    const uint2 lo = *reinterpret_cast<const uint2 *>(b + (rowbyte + 2u * (uint32_t)(32 * h + 4 * g)));
    const uint2 hi = *reinterpret_cast<const uint2 *>(b + (rowbyte + 2u * (uint32_t)(32 * h + 16 + 4 * g)));
    return make_bf16x8(lo.x, lo.y, hi.x, hi.y);
}
__device__ __forceinline__ s16x4 pack4(const f32x4 &a) {
    return make_s16x4(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]));
}
__device__ __forceinline__ void unpack4(const s16x4 &a, float (&o)[4]) {
    const u32x2 t = __builtin_bit_cast(u32x2, a);
    o[0] = __uint_as_float(t[0] << 16); o[1] = __uint_as_float(t[0] & 0xffff0000u);
    o[2] = __uint_as_float(t[1] << 16); o[3] = __uint_as_float(t[1] & 0xffff0000u);
}
__device__ __forceinline__ void unpack8(const bf16x8 &a, float (&o)[8]) {
    const u32x4 t = __builtin_bit_cast(u32x4, a);
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(t[i] << 16); o[2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u); }
}


// The chunked kernels take bf16 tensors (outputs bf16) or fp16 tensors (outputs fp32, the reference's
// rule for half inputs).  r, k, w go through fp32 code anyway, so their 16-bit tiles are unpacked as
// what they are; v and gy are consumed as bf16 MFMA operands, so for fp16 tensors the caller passes
// bf16 copies of them (and the originals for the exact per-timestep pass).
template <typename Tin> struct OutOf { typedef bf16_t type; };
template <> struct OutOf<f16_t> { typedef float type; };
template <typename Tin> __device__ __forceinline__ float in_bits_to_float(uint32_t bits);
template <> __device__ __forceinline__ float in_bits_to_float<bf16_t>(uint32_t bits) { return __uint_as_float(bits << 16); }
template <> __device__ __forceinline__ float in_bits_to_float<f16_t>(uint32_t bits) { return (float)__builtin_bit_cast(f16_t, (uint16_t)bits); }
template <typename Tin> constexpr uint32_t neg_inf_bits() { return 0xff80u; }
template <> constexpr uint32_t neg_inf_bits<f16_t>() { return 0xfc00u; }
// four consecutive 16-bit elements of the input type (as read from a tile) -> fp32
template <typename Tin> __device__ __forceinline__ void unpack4_in(const s16x4 &a, float (&o)[4]);
template <> __device__ __forceinline__ void unpack4_in<bf16_t>(const s16x4 &a, float (&o)[4]) { unpack4(a, o); }
template <> __device__ __forceinline__ void unpack4_in<f16_t>(const s16x4 &a, float (&o)[4]) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 x = __builtin_bit_cast(h4, a);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (float)x[i];
}

// ------------------------------------------------------------------------------------------
// LDS tiles: bf16 [token][64 channels], 128-byte rows, no padding; the eight 16-byte pieces of a
// row are XOR-swizzled with (token & 7).  One layout serves the loads that fill a tile straight
// from global memory, the lane = channel accesses of the operand preparation, and both MFMA
// fragment orientations (the second through the transposing LDS read of gfx950).
// ------------------------------------------------------------------------------------------
constexpr int kTileRow = 128;                 // bytes per token row
constexpr int kTileBytes = 64 * kTileRow;     // one 64-token chunk of one tensor

__device__ __forceinline__ uint32_t tile_off(int t, int ch) {
    return ((uint32_t)t << 7) + (((((uint32_t)ch >> 3) ^ (uint32_t)t) & 7u) << 4) + (((uint32_t)ch & 7u) << 1);
}

// Eight token rows (t0 .. t0+7 of the tile, t0 a multiple of 8) of one head's 128-byte row
// segments, global -> LDS without passing through registers: lane L brings the 16-byte piece that
// belongs at LDS position 16 L of the block.  `voff` is the lane's byte offset from the uniform
// `gbase` (row (L >> 3), piece ((L & 7) ^ (L >> 3))); `lds_addr` the uniform LDS byte address of
// row t0.  Completion is counted by vmcnt; the compiler does not know about these loads, so the
// caller waits with wait_loads<N>() (N = number of younger loads allowed to stay in flight).
__device__ __forceinline__ void load_rows8_to_lds(const void *gbase, uint32_t voff, uint32_t lds_addr) {
    // (the uniform operands are pinned to scalar registers explicitly: an "s" constraint alone does
    // not move a value the compiler happened to keep in vector registers)
    const uint64_t gb = reinterpret_cast<uint64_t>(gbase);
    const uint32_t ub_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)gb);          // (the builtin returns a
    const uint32_t ub_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(gb >> 32));   //  signed int: no widening casts)
    const uint64_t ub = ((uint64_t)ub_hi << 32) | (uint64_t)ub_lo;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(ub) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

// a wave-uniform value the compiler has to treat as newly defined (it stays in a scalar register)
__device__ __forceinline__ int fresh_s(int x) { asm volatile("" : "+s"(x)); return x; }

__device__ __forceinline__ uint32_t lds_address(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char *)p;
}

// A/B fragment with the k-slots along the CHANNELS of token `row`, for one 16x16x32 MFMA over
// channels [32h, 32h+32): k-slots {32h+4g+e, 32h+16+4g+e : e<4} (the order acc_as_operand produces).
__device__ __forceinline__ bf16x8 tile_frag_ch(const unsigned char *tile, int row, int h, int g) {
    const uint2 lo = *reinterpret_cast<const uint2 *>(tile + tile_off(row, 32 * h + 4 * g));
    const uint2 hi = *reinterpret_cast<const uint2 *>(tile + tile_off(row, 32 * h + 16 + 4 * g));
    return make_bf16x8(lo.x, lo.y, hi.x, hi.y);
}
// A/B fragment with the k-slots along the TOKENS, for one 16x16x16 MFMA: the lane (l16, g) of the
// result holds tile[tk0 + 4g + e][n0 + l16], e < 4.  (The transposing read hands lane l16 of a
// 16-lane group the l16-th element of each of four 16-element rows; row e is assembled from the
// 8-byte pieces that lanes 4e..4e+3 of the group point at.)
__device__ __forceinline__ s16x4 tile_frag_tok(const unsigned char *tile, int n0, int tk0, int l16, int g) {
    const unsigned char *p = tile + tile_off(tk0 + 4 * g + (l16 >> 2), n0 + 4 * (l16 & 3));
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
}

}  // namespace wkv6
