// Shared pieces of the block-form WKV6 kernels (wkv6_block_fwd.hip, wkv6_block_bwd.hip).
//
// Block form: a chunk visit covers 64 tokens = two blocks of 32; a block is one step of the state
// recurrences.  Inside a block the decay exponents are taken relative to the block's MIDDLE token
// (c_t = running sum of exp(w); alpha_t = exp(-(c_t - c_mid))), so the scaled operands
//   R~_t = r_t alpha_t,   K~_s = k_s / alpha_{s+1}
// stay within exp(+-sum of exp(w) over 16 tokens) -- the same range the tile form has (16-token tiles
// scaled from the tile start), and the same range check per 16 tokens.  With
//   g1 = exp(-(c_mid - c_first)),  g2 = exp(-(c_end - c_mid))
// a state S entering a block acts through g1 o S, and leaves it as g2 o (g1 o S + K~^T V).
#pragma once
#include "wkv6_mfma.h"

namespace wkv6 {

constexpr int kBlockTokens = 64;                      // tokens per chunk visit (two blocks of 32)
constexpr int kBlockMaxSlots = 64;   // (batch, head) pairs one workgroup takes at most
constexpr float kLog2Log2e = 0.5287663729448977f;     // log2(log2(e)): exp(w) log2(e) = 2^(w log2(e) + this)

// Per-visit vectors the producer waves leave for the others: [g1 of block 0, g2 of block 0, g1 of
// block 1, g2 of block 1, diagonal sum r u k of the 64 tokens], 64 floats each.  Producer wave p
// (tokens 16p..16p+15) owns row p: the first 16 tokens of a block give its g1, the last 16 its g2.
constexpr int kBlockVecBytes = 5 * kN * 4;

// ------------------------------------------------------------------------------------------
// Fragments with the k-slots along the channels in CONTIGUOUS order: lane group g of a 16x16x32 MFMA
// takes k-slots 32h + 8g .. 32h + 8g + 7, one 16-byte LDS read per fragment (half the instructions of
// the two 8-byte reads of tile_frag_ch, and no bank conflicts between rows t and t + 8).
// An accumulator stack reused as such an operand (acc_as_operand(S[2h], S[2h+1])) must then hold, in
// accumulator m, row 4g + rr, the channel  32 (m >> 1) + 8g + 4 (m & 1) + rr  -- block_row_channel().
// That is arranged by the rows of the operand that PRODUCES the accumulator (block_frag_tok_rows).
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ bf16x8 block_frag_ch(const unsigned char *tile, int row, int h, int g) {
    const uint4 x = *reinterpret_cast<const uint4 *>(tile + tile_off(row, 32 * h + 8 * g));
    return make_bf16x8(x.x, x.y, x.z, x.w);
}
// first of the four channels accumulator m holds in lane group g
__device__ __forceinline__ int block_row_channel(int m, int g) { return 32 * (m >> 1) + 8 * g + 4 * (m & 1); }
// A/B fragment with the k-slots along the TOKENS tk0 + 4g + e (e < 4) for one 16x16x16 MFMA whose 16
// rows (lane l16) are the channels accumulator m is to hold: row l16 <-> channel block_row_channel(m, l16 >> 2) + (l16 & 3).
__device__ __forceinline__ s16x4 block_frag_tok_rows(const unsigned char *tile, int m, int tk0, int l16, int g) {
    const unsigned char *p = tile + tile_off(tk0 + 4 * g + (l16 >> 2), 32 * (m >> 1) + 8 * (l16 & 3) + 4 * (m & 1));
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
}
// The transposed state tile ([i][j] rows of 128 bytes): S[j = n0 + l16][i = block_row_channel(m, g) + e], e < 4
__device__ __forceinline__ u32x2 block_state_frag(const unsigned char *tile, int n0, int m, int l16, int g) {
    const unsigned char *p = tile + tile_off(block_row_channel(m, g) + (l16 >> 2), n0 + 4 * (l16 & 3));
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p));
}

// ------------------------------------------------------------------------------------------
// The same addresses from a handful of per-lane bases.  tile_off() mixes the row into the piece index
// with an XOR, so the compiler cannot see that the offsets of a fragment for different row groups,
// channel halves or accumulators differ by constants, and keeps dozens of them in registers.  Spelled
// out: every address below is  (lane base ^ small constant) + immediate.
//   row groups of 16 (or 8) tokens: + 128 * first row (immediate);
//   the other half of the channels (h = 1), accumulators 2 and 3: piece index ^ 4  = offset ^ 64;
//   column block n0 = 16 n of a token-wise fragment: piece index ^ 2n = offset ^ 32 n.
// ------------------------------------------------------------------------------------------
struct BlockLane {
    uint32_t ch;     // block_frag_ch: row l16, channels 8g (h = 0)
    uint32_t tok;    // tile_frag_tok, n0 = 0: row 4g + (l16 >> 2), channels 4 (l16 & 3)
    uint32_t rows;   // block_frag_tok_rows, m = 0: row 4g + (l16 >> 2), channels 8 (l16 & 3)
    __device__ __forceinline__ BlockLane(int l16, int g) {
        const uint32_t r = (uint32_t)(4 * g + (l16 >> 2));
        ch = ((uint32_t)l16 << 7) + ((((uint32_t)g ^ (uint32_t)l16) & 7u) << 4);
        tok = (r << 7) + ((((((uint32_t)l16 >> 1) & 1u) ^ r) & 7u) << 4) + (((uint32_t)l16 & 1u) << 3);
        rows = (r << 7) + (((((uint32_t)l16 & 3u) ^ r) & 7u) << 4);
    }
    // fragment with the k-slots along channels 32h + 8g .. +7 of token row0 + l16 (row0 a multiple of 8)
    __device__ __forceinline__ bf16x8 frag_ch(const unsigned char *tile, int row0, int h) const {
        const uint4 x = *reinterpret_cast<const uint4 *>(tile + (ch ^ (uint32_t)(h << 6)) + row0 * kTileRow);
        return make_bf16x8(x.x, x.y, x.z, x.w);
    }
    // tile[tk0 + 4g + e][16 n + l16], e < 4 (tk0 a multiple of 8)
    __device__ __forceinline__ s16x4 frag_tok(const unsigned char *tile, int n, int tk0) const {
        const unsigned char *p = tile + (tok ^ (uint32_t)(n << 5)) + tk0 * kTileRow;
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
    }
    // tile[tk0 + 4g + e][channel of row l16 of accumulator m], e < 4
    __device__ __forceinline__ s16x4 frag_tok_rows(const unsigned char *tile, int m, int tk0) const {
        const unsigned char *p = tile + (rows ^ (uint32_t)((m >> 1) << 6)) + ((m & 1) << 3) + tk0 * kTileRow;
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
    }
    // offset of channels block_row_channel(m, g) .. +3 in the row row0 + l16 (8-byte accesses: a lane's four accumulator rows)
    __device__ __forceinline__ uint32_t acc_rows_off(int m, int row0) const {
        return (ch ^ (uint32_t)((m >> 1) << 6)) + ((m & 1) << 3) + row0 * kTileRow;
    }
};
// offset of channels 16q + 4g .. +3 in row l16 of a row group (add 128 * first row): the elementwise
// pass and the staging of transposed products
__device__ __forceinline__ uint32_t block_lane_cols4(int q, int l16, int g) {
    return ((uint32_t)l16 << 7) + ((((uint32_t)(2 * q + (g >> 1)) ^ (uint32_t)l16) & 7u) << 4) + (((uint32_t)g & 1u) << 3);
}
// the transposed state tile: S[j = 16q + l16][i = block_row_channel(m, g) + e]: base for m = 0; m: ^ 64 (m & 1), + 128 (32 (m >> 1) + 4 (m & 1))
__device__ __forceinline__ uint32_t block_lane_state(int q, int l16, int g) {
    const uint32_t r = (uint32_t)(l16 >> 2);
    return ((uint32_t)(8 * g) + r) * 128u + ((((uint32_t)(2 * q) | (((uint32_t)l16 >> 1) & 1u)) ^ r) << 4) + (((uint32_t)l16 & 1u) << 3);
}
__device__ __forceinline__ u32x2 block_state_frag_at(const unsigned char *tile, uint32_t lane_state, int m) {
    const unsigned char *p = tile + (lane_state ^ (uint32_t)((m & 1) << 6)) + (32 * (m >> 1) + 4 * (m & 1)) * kTileRow;
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p));
}

// sum over the 16 lanes of a row (result in every lane of the row)
__device__ __forceinline__ float sum_row16(float x) {
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));   // row_half_mirror
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x140, 0xF, 0xF, true));   // row_mirror
    return x;
}

// Waits until at most n of this wave's vector-memory operations are still in flight (n even; the
// instruction takes the count as an immediate, so the nearest immediate at or below n is used).
__device__ __forceinline__ void wait_in_flight(int n) {
    if (n >= 32) wait_loads<32>();
    else if (n >= 28) wait_loads<28>();
    else if (n >= 24) wait_loads<24>();
    else if (n >= 22) wait_loads<22>();
    else if (n >= 20) wait_loads<20>();
    else if (n >= 18) wait_loads<18>();
    else if (n >= 16) wait_loads<16>();
    else if (n >= 14) wait_loads<14>();
    else if (n >= 12) wait_loads<12>();
    else if (n >= 10) wait_loads<10>();
    else if (n >= 8) wait_loads<8>();
    else if (n >= 6) wait_loads<6>();
    else if (n >= 4) wait_loads<4>();
    else if (n >= 2) wait_loads<2>();
    else wait_loads<0>();
}

// Two 16-token row groups, each lane holding four channels (8 bytes: `a` of the first group's token l16,
// `b` of the second group's) -> one 16-byte piece per lane: lanes of even g receive the channels
// 4g .. 4g+7 of the first group's token, lanes of odd g the channels 4(g-1) .. 4g+3 of the second
// group's (rows of 16 lanes are swapped between the two registers).
__device__ __forceinline__ u32x4 pair_rows_8ch(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1)
{
    const auto x = __builtin_amdgcn_permlane16_swap(a0, b0, false, false);
    const auto y = __builtin_amdgcn_permlane16_swap(a1, b1, false, false);
    return (u32x4){x[0], y[0], x[1], y[1]};
}

// Operand preparation of one producer wave (tokens 16p .. 16p+15 of a chunk; lane (l16, g) holds
// channels 4 l16 .. +3 of tokens 4g .. 4g+3, all LDS accesses 8 bytes wide).  Reads the raw r, k, w
// rows, leaves the per-visit vectors of this wave (its g1 or g2 row, its 16 diagonal sums) and hands
// every element's scaled values to `emit(o, xr, xk, alpha_next, ew2)`: o the tile offset of the
// lane's four channels in the row of token 4g + e, xr / xk = R~ / K~, alpha_next = alpha_{t+1},
// ew2 = exp(w) log2(e).  Returns false if the wave's 16 tokens leave the range the scaled operands
// can hold (any channel).
// `after_read()` runs once the raw rows are in registers (their LDS block may be refilled from then on).
// kRagged: only the first `valid` tokens of the chunk exist; the others are prepared as r = k = 0 with
// decay 1 (exp(w) = 0), so that they leave both states alone and contribute nothing (their rows hold
// copies of the last token that exists).
template <bool kRagged, typename AfterRead, typename Emit>
__device__ __forceinline__ bool block_prepare(const unsigned char *raw_r, const unsigned char *raw_k, const unsigned char *raw_w,
                                              float *vec, const float (&u4)[4], int p, int l16, int g, int valid, AfterRead after_read, Emit emit)
{
    uint2 qr[4], qk[4], qw[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t o = tile_off(16 * p + 4 * g + e, 4 * l16);
        qr[e] = *reinterpret_cast<const uint2 *>(raw_r + o);
        qk[e] = *reinterpret_cast<const uint2 *>(raw_k + o);
        qw[e] = *reinterpret_cast<const uint2 *>(raw_w + o);
    }
    after_read();
    float fr[4][4], fk[4][4], ew2[4][4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float fw[4];
        unpack4(make_s16x4(qr[e].x, qr[e].y), fr[e]);
        unpack4(make_s16x4(qk[e].x, qk[e].y), fk[e]);
        unpack4(make_s16x4(qw[e].x, qw[e].y), fw);
#pragma unroll
        for (int c = 0; c < 4; ++c) ew2[e][c] = exp2_fast(fmaf(fw[c], kLog2e, kLog2Log2e));   // exp(w) log2(e): exponents in base 2
        if (kRagged && 16 * p + 4 * g + e >= valid) {
#pragma unroll
            for (int c = 0; c < 4; ++c) { fr[e][c] = 0.f; fk[e][c] = 0.f; ew2[e][c] = 0.f; }
        }
    }
    // running sums: inside the lane (4 tokens), across the four lane groups; relative to the block's
    // middle, which is the END of an even wave's tokens and the START of an odd wave's
    float ex[4], tot[4];
    bool ok = true;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float lt = (ew2[0][c] + ew2[1][c]) + (ew2[2][c] + ew2[3][c]);
        tot[c] = sum_rows(lt);
        ex[c] = prefix_rows(lt, g) - ((p & 1) ? 0.f : tot[c]);
        ok = ok && (tot[c] <= kWildLimit * kLog2e);
    }
    if (g == 0)
        *reinterpret_cast<float4 *>(&vec[p * kN + 4 * l16]) =
            make_float4(exp2_fast(-tot[0]), exp2_fast(-tot[1]), exp2_fast(-tot[2]), exp2_fast(-tot[3]));
    {
        // the diagonal of A: sum over the channels of r u k, one value per token
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            d[e] = (fr[e][0] * u4[0] * fk[e][0] + fr[e][1] * u4[1] * fk[e][1]) + (fr[e][2] * u4[2] * fk[e][2] + fr[e][3] * u4[3] * fk[e][3]);
#pragma unroll
        for (int e = 0; e < 4; ++e) d[e] = sum_row16(d[e]);
        if (l16 == 0) *reinterpret_cast<float4 *>(&vec[4 * kN + 16 * p + 4 * g]) = make_float4(d[0], d[1], d[2], d[3]);
    }
    float al[4];   // alpha_t of the lane's current token (the previous token's alpha_{t+1})
#pragma unroll
    for (int c = 0; c < 4; ++c) al[c] = exp2_fast(-ex[c]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float xr[4], xk[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            xr[c] = fr[e][c] * al[c];
            ex[c] += ew2[e][c];
            al[c] = exp2_fast(-ex[c]);   // alpha_{t+1}
            xk[c] = fk[e][c] * exp2_fast(ex[c]);
        }
        emit(tile_off(16 * p + 4 * g + e, 4 * l16), xr, xk, al, ew2[e]);
    }
    return __builtin_amdgcn_ballot_w64(!ok) == 0ull;
}

}  // namespace wkv6
