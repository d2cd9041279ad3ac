// WKV6 in chunk-parallel form for gfx950: bf16 MFMA for the dense products, fp32 state.
//
// One workgroup (8 waves) per (batch, head).  Time is cut into chunks of 64 tokens, each chunk
// into 4 tiles of 16 tokens.  The fp32 state S[j][i] lives in the MFMA accumulators of the four
// "consumer" waves (wave q owns value columns 16q..16q+15) and is advanced one tile at a time:
//
//   c_t = sum_{s<t} exp(w_s) inside the tile (so exp(-c_t) is the decay from the tile start to t)
//   R~[t][j] = r_t[j] exp(-c_t[j])            K~[t][j] = k_t[j] exp(+c_{t+1}[j])
//   K^[t][j] = k_t[j] exp(-(c_16[j] - c_{t+1}[j]))         g[j] = exp(-c_16[j])
//   A[t][s]  = R~_t . K~_s  (s < t),  A[t][t] = sum_j r_t[j] u[j] k_t[j]
//   Y        = R~ S + A V          (16x64x64 and 16x16x16 MFMA, K index j resp. s)
//   S       <- diag(g) S + K^T V   (64x16x16 MFMA, K index s)
//
// The four "producer" waves (wave 4+p prepares tile p, lane = channel) compute these operands in
// fp32 for the NEXT chunk while the consumers run the MFMAs of the current one; LDS operand
// buffers are double-buffered and the two roles meet at one barrier per chunk.  HBM traffic is
// exactly the algorithmic minimum (r,k,v,w read once, y written once).
//
// exp(+c) needs the decay accumulated inside one 16-token tile to stay in range.  A producer wave
// that meets a tile whose summed exp(w) exceeds kWildLimit in any channel raises a flag in LDS, and
// the workgroup then redoes ITS (batch, head) pair with the exact per-timestep code
// (wkv6_scan_body.h) before the kernel ends; other workgroups are unaffected.
#include "wkv6_common.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>

namespace wkv6 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int CL = 64;   // tokens per chunk
constexpr int LDA = 68;  // row pitch (elements) of [token][channel] operand arrays: 136 B, conflict-free 8-byte fragment reads
constexpr int LDT = 72;  // row pitch (elements) of [channel][token] operand arrays: 144 B, 16-byte aligned rows
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

// 16-bit load at a uniform base + 32-bit per-lane byte offset (lets the compiler use the
// scalar-base addressing form instead of 64-bit per-lane address arithmetic)
__device__ __forceinline__ uint32_t ld16(const void *base, uint32_t byteoff) {
    return *reinterpret_cast<const uint16_t *>(reinterpret_cast<const char *>(base) + byteoff);
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
__device__ __forceinline__ s16x4 frag_ct(const uint16_t (*a)[LDT], int ch, int tok) {
    const uint2 x = *reinterpret_cast<const uint2 *>(&a[ch][tok]);
    return make_s16x4(x.x, x.y);
}
// two accumulator tiles (rows 16m+4g+r and 16(m+1)+4g+r) as the bf16 operand of a 16x16x32 MFMA
__device__ __forceinline__ bf16x8 acc_as_operand(const f32x4 &a, const f32x4 &b) {
    return make_bf16x8(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(b[0], b[1]), pack_bf16x2(b[2], b[3]));
}

// sum over the 64 lanes of 16 per-lane values; lane l receives the total of value (l>>2)&15
__device__ __forceinline__ float transpose_reduce16(const float (&p)[16], int lane) {
    float x8[8], x4[4], x2[2];
    const bool b5 = lane & 32, b4 = lane & 16, b3 = lane & 8, b2 = lane & 4;
#pragma unroll
    for (int a = 0; a < 8; ++a) x8[a] = (b5 ? p[a + 8] : p[a]) + __shfl_xor(b5 ? p[a] : p[a + 8], 32);
#pragma unroll
    for (int a = 0; a < 4; ++a) x4[a] = (b4 ? x8[a + 4] : x8[a]) + __shfl_xor(b4 ? x8[a] : x8[a + 4], 16);
#pragma unroll
    for (int a = 0; a < 2; ++a) x2[a] = (b3 ? x4[a + 2] : x4[a]) + __shfl_xor(b3 ? x4[a] : x4[a + 2], 8);
    float x = (b2 ? x2[1] : x2[0]) + __shfl_xor(b2 ? x2[0] : x2[1], 4);
    x += __shfl_xor(x, 2);
    x += __shfl_xor(x, 1);
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

struct alignas(16) FwdBuf {
    uint16_t rt[CL][LDA];   // R~[t][j]
    uint16_t kt[CL][LDA];   // K~[t][j]
    uint16_t ktT[kN][LDT];  // K~[t][j] stored [j][t]  (K^ = g K~ is never formed: S <- g (S + K~^T V))
    uint16_t vT[kN][LDT];   // V[t][i]  stored [i][t]
    float g[4][kN];         // per-tile decay exp(-c_16)
    float ruk[CL];          // sum_j r u k per token
};

// kSave: also write the state at every chunk start to `ckpt` (fp32, [b][h][chunk][j][i]) for the
// backward pass, which then skips its own forward sweep.
template <typename Ts, bool kSave, bool kRagged>
__global__ __launch_bounds__(512) void chunk_fwd_kernel(int T, int H,
        const bf16_t *__restrict__ r, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v,
        const bf16_t *__restrict__ w, const bf16_t *__restrict__ u,
        const Ts *__restrict__ s0, const int64_t *__restrict__ map,
        bf16_t *__restrict__ y, Ts *__restrict__ sT, float *__restrict__ ckpt)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild;
    FwdBuf *buf = reinterpret_cast<FwdBuf *>(smem);
    static_assert(sizeof(ScanFwdLds) <= 2 * sizeof(FwdBuf), "the exact second pass reuses the operand buffers");
    if (threadIdx.x == 0) s_wild = 0;
    __syncthreads();

    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
    const int nchunk = (T + CL - 1) / CL;

    if (wave < 4) {
        // ------------------------------ consumer: MFMA ------------------------------
        const int q = wave, g = lane >> 4, l16 = lane & 15;
        f32x4 S[4];
        if (s0 != nullptr) {
            const int64_t row = map ? map[b] : (int64_t)b;
            const Ts *p = s0 + (row * H + h) * kN * kN + 16 * q + l16;
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) S[m][rr] = load1(p + (16 * m + 4 * g + rr) * kN);
        } else {
#pragma unroll
            for (int m = 0; m < 4; ++m) S[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        bf16_t *y_h = y + base;
        for (int c = 0; c < nchunk; ++c) {
            if (kSave) {
                float *dst = ckpt + ((int64_t)blockIdx.x * nchunk + c) * (kN * kN) + 16 * q + l16;
#pragma unroll
                for (int m = 0; m < 4; ++m)
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) dst[(16 * m + 4 * g + rr) * kN] = S[m][rr];
            }
            __syncthreads();
            const FwdBuf &B = buf[c & 1];
            const int t0 = c * CL;
#pragma unroll 1
            for (int p = 0; p < 4; ++p) {
                if (t0 + 16 * p >= T) break;
                const int row = 16 * p + l16;
                const bf16x8 rf0 = frag_tc(B.rt, row, 0, g), rf1 = frag_tc(B.rt, row, 1, g);
                const bf16x8 kf0 = frag_tc(B.kt, row, 0, g), kf1 = frag_tc(B.kt, row, 1, g);
                const s16x4 vf = frag_ct(B.vT, 16 * q + l16, 16 * p + 4 * g);
                const float rukv = B.ruk[row];
                // A^T[s][t] = K~_s . R~_t  (accumulator rows s = 4g+r, column t = l16)
                f32x4 AT = {0.f, 0.f, 0.f, 0.f};
                AT = mfma32(kf0, rf0, AT);
                AT = mfma32(kf1, rf1, AT);
                // Y = R~ S
                f32x4 Y = {0.f, 0.f, 0.f, 0.f};
                Y = mfma32(rf0, acc_as_operand(S[0], S[1]), Y);
                Y = mfma32(rf1, acc_as_operand(S[2], S[3]), Y);
                settle(AT);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int s = 4 * g + rr;
                    AT[rr] = (l16 > s) ? AT[rr] : ((l16 == s) ? rukv : 0.f);
                }
                // Y += A V : the masked A^T accumulator IS the A operand (row t = l16, k-slots s = 4g+r)
                chain_gap(Y);
                Y = mfma16(make_s16x4(pack_bf16x2(AT[0], AT[1]), pack_bf16x2(AT[2], AT[3])), vf, Y);
                // S <- diag(g) (S + K~^T V)
#pragma unroll
                for (int m = 0; m < 4; ++m) S[m] = mfma16(frag_ct(B.ktT, 16 * m + l16, 16 * p + 4 * g), vf, S[m]);
                settle(Y, S[0], S[1], S[2], S[3]);   // Y is stored, S scaled and converted by VALU code from here on
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 gg = *reinterpret_cast<const float4 *>(&B.g[p][16 * m + 4 * g]);
                    S[m][0] *= gg.x; S[m][1] *= gg.y; S[m][2] *= gg.z; S[m][3] *= gg.w;
                }
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int t = t0 + 16 * p + 4 * g + rr;
                    if (!kRagged || t < T) st16(y_h, (uint32_t)t * (uint32_t)C * 2u + 2u * (uint32_t)(16 * q + l16), Y[rr]);
                }
            }
        }
        if (sT != nullptr) {
            Ts *p = sT + ((int64_t)b * H + h) * kN * kN + 16 * q + l16;
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) store1(p + (16 * m + 4 * g + rr) * kN, S[m][rr]);
        }
    } else {
        // ------------------------------ producer: operand preparation ------------------------------
        const int p = wave - 4, ch = lane;
        const float uc = load1(u + h * kN + ch);
        const bf16_t *rb = r + base, *kb_ = k + base, *vb = v + base, *wb = w + base;   // uniform
        const uint32_t rowbytes = (uint32_t)C * 2u;
        uint32_t qr[16], qk[16], qv[16], qw[16];
        // Tokens past the end read as r = k = v = 0, w = -inf (exp(w) = 0, decay 1).  Without kRagged
        // a tile is either entirely inside the sequence or entirely outside.
        auto prefetch = [&](int c) {
            const int tb = c * CL + 16 * p;
            if (tb < T) {   // uniform: a tile entirely past the end is neither loaded, prepared nor consumed
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int t = tb + e;
                    const bool ok = !kRagged || t < T;
                    const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + 2u * (uint32_t)ch;
                    const uint32_t a = ld16(rb, o), bb = ld16(kb_, o), cc = ld16(vb, o), dd = ld16(wb, o);
                    qr[e] = ok ? a : 0u; qk[e] = ok ? bb : 0u; qv[e] = ok ? cc : 0u; qw[e] = ok ? dd : 0xff80u;
                }
            }
        };
        auto prepare = [&](int c) {   // consumes the prefetched registers, refills them for chunk c+1
            FwdBuf &B = buf[c & 1];
            const bool tile_in = c * CL + 16 * p < T;
            float fr[16], fk[16], fw[16];
            uint32_t vbits[8];
            if (tile_in) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    fr[e] = bf16_bits_to_float(qr[e]); fk[e] = bf16_bits_to_float(qk[e]); fw[e] = bf16_bits_to_float(qw[e]);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) vbits[e] = qv[2 * e] | (qv[2 * e + 1] << 16);
            }
            if (c + 1 < nchunk) prefetch(c + 1);
            if (tile_in) {

            // exponents are kept in base 2 (one v_exp_f32 each, no extra scaling multiply)
            float xr[16], xk[16], pr[16];
            float cs2 = 0.f, pa = 1.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float ew2 = exp2_fast(fw[e] * kLog2e) * kLog2e;   // exp(w) * log2(e)
                xr[e] = fr[e] * pa;               // r exp(-c_t)
                cs2 += ew2;
                xk[e] = fk[e] * exp2_fast(cs2);   // k exp(+c_{t+1})
                pa *= exp2_fast(-ew2);
                pr[e] = fr[e] * uc * fk[e];
            }
            if (__builtin_amdgcn_ballot_w64(!(cs2 <= kWildLimit * kLog2e)) != 0ull) {
                if (lane == 0) s_wild = 1;
            }
            store_rows_paired(B.rt, 16 * p, lane, xr);
            store_rows_paired(B.kt, 16 * p, lane, xk);
            uint32_t kb[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) kb[e] = pack_bf16x2(xk[2 * e], xk[2 * e + 1]);
            *reinterpret_cast<uint4 *>(&B.ktT[ch][16 * p]) = make_uint4(kb[0], kb[1], kb[2], kb[3]);
            *reinterpret_cast<uint4 *>(&B.ktT[ch][16 * p + 8]) = make_uint4(kb[4], kb[5], kb[6], kb[7]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p]) = make_uint4(vbits[0], vbits[1], vbits[2], vbits[3]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p + 8]) = make_uint4(vbits[4], vbits[5], vbits[6], vbits[7]);
            B.g[p][ch] = pa;
            const float tot = transpose_reduce16(pr, lane);
            if ((lane & 3) == 0) B.ruk[16 * p + ((lane >> 2) & 15)] = tot;
            }
        };
        prefetch(0);
        prepare(0);
        for (int c = 0; c < nchunk; ++c) {
            __syncthreads();
            if (c + 1 < nchunk) prepare(c + 1);
        }
    }
    // exact second pass for this (b, h) if any of its tiles left the representable range
    __threadfence_block();   // workgroup scope is enough (and a device-scope fence would write back the L2)
    __syncthreads();
    if (s_wild)
        scan_fwd_body<bf16_t, bf16_t, Ts>(*reinterpret_cast<ScanFwdLds *>(smem), b, h, T, H, r, k, v, w, u, s0, map, y, sT);
}

// ==========================================================================================
// Backward.
//
// Same workgroup shape as the forward kernel.  Phase 1 sweeps the chunks in time order and writes
// the state at every chunk start to the workspace (fp32, [b][h][chunk][j][i]); phase 2 sweeps them
// in reverse order with the reverse state G in the accumulators.  G is kept twice, once with rows j
// / columns i (for gv) and once transposed (for gk), so that it can be fed back to the MFMAs as an
// operand without leaving the registers; the forward state at each of the 4 tile starts of a chunk
// is recomputed from the checkpoint and held as packed bf16 operands.
//
// Per tile (16 tokens; t, s local token indices; c as in the forward kernel; G = reverse state
// entering the tile from the future, S0 = forward state at the tile start):
//   dA[t][s] = gy_t . v_s (s<t)                       A[t][s] = R~_t . K~_s (s<t),  A[t][t] = sum_j r u k
//   X[t][j]  = sum_s dA[t][s] K~_s[j] + sum_i gy_t[i] S0[j][i]        gr'_t[j] = exp(-c_t) X,   P = R~ X
//   W[s][j]  = sum_t dA[t][s] R~_t[j] + g_j sum_i v_s[i] G[j][i]      gk'_s[j] = exp(+c_{s+1}) W, Q = K~ W
//   gv_s[i]  = sum_t A[t][s] gy_t[i] + sum_j K~_s[j] g_j G[j][i]
//   G       <- diag(g) G + R~^T gY
//   gr = gr' + u k <v,gy>,  gk = gk' + u r <v,gy>,  gu[j] = sum_t r k <v,gy>
//   gw_t[j]  = -exp(w_t[j]) ( E[j] + sum_{m<t} (Q_m - P_m) - P_t ),  E[j] = sum_i S0[j][i] G_new[j][i]
// (the last line is the flow balance across decay step t, anchored at the exact tile-boundary term E).
// ==========================================================================================
constexpr int LDFR = 80;  // floats per channel row of the decay-factor array: 4 tiles x (17 used + 3 pad)

struct alignas(16) BwdBuf {
    uint16_t rt[CL][LDA];    // R~[t][j]
    uint16_t kt[CL][LDA];    // K~[t][j]
    uint16_t rtT[kN][LDT];   // R~ stored [j][t]
    uint16_t ktT[kN][LDT];   // K~ stored [j][t]
    uint16_t vT[kN][LDT];    // V  stored [i][t]
    uint16_t gyT[kN][LDT];   // gY stored [i][t]
    float fr[kN][LDFR];      // fr[j][20p + t] = exp(-c_t) of tile p, t = 0..16
    float g[4][kN];
    float ruk[CL];
    float vgyw[4][16];       // <v_t, gy_t> of the tile in flight, one private copy per consumer wave
};

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

// operand number p of four, p uniform over the wave; dword-wise selects keep everything in registers
__device__ __forceinline__ bf16x8 pick4(const bf16x8 &a0, const bf16x8 &a1, const bf16x8 &a2, const bf16x8 &a3, int p) {
    const u32x4 x0 = __builtin_bit_cast(u32x4, a0), x1 = __builtin_bit_cast(u32x4, a1);
    const u32x4 x2 = __builtin_bit_cast(u32x4, a2), x3 = __builtin_bit_cast(u32x4, a3);
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = (p == 1) ? x1[i] : x0[i];
        const uint32_t hi = (p == 3) ? x3[i] : x2[i];
        o[i] = (p >= 2) ? hi : lo;
    }
    return make_bf16x8(o[0], o[1], o[2], o[3]);
}

// kRagged: T is not a multiple of 16, so the last tile has rows past the end.  The common
// kRagged = false build has no per-lane predicates in the tile loops at all: with them every tile
// body splits into several basic blocks, the compiler sinks the early-issued loads back next to
// their uses and, since vmcnt is a single in-order counter, makes each tile wait for the previous
// tile's stores to be acknowledged.
#ifdef WKV6_TIMING
#define WKV6_STAMP() do { if (blockIdx.x == 0 && lane == 0 && dbg_n < 250) dbg[wave * 256 + dbg_n++] = __builtin_readcyclecounter(); } while (0)
#else
#define WKV6_STAMP() do { } while (0)
#endif

template <bool kSweepStates, bool kRagged>
__global__ __launch_bounds__(512) void chunk_bwd_kernel(int T, int H,
        const bf16_t *__restrict__ r, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v,
        const bf16_t *__restrict__ w, const bf16_t *__restrict__ u, const bf16_t *__restrict__ gy,
        bf16_t *__restrict__ gr, bf16_t *__restrict__ gk, bf16_t *__restrict__ gv, bf16_t *__restrict__ gw,
        bf16_t *__restrict__ gu, float *__restrict__ ckpt)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild;
    BwdBuf *buf = reinterpret_cast<BwdBuf *>(smem);
    static_assert(sizeof(ScanBwdALds) <= 2 * sizeof(BwdBuf) && sizeof(ScanBwdBLds) <= 2 * sizeof(BwdBuf),
                  "the exact second pass reuses the operand buffers");
    if (threadIdx.x == 0) s_wild = 0;
    __syncthreads();

    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
    const int nchunk = (T + CL - 1) / CL;
    const int nitem = kSweepStates ? 2 * nchunk : nchunk;   // work items: [phase 1 chunks 0..n-1] then phase 2 chunks n-1..0
    float *ck = ckpt + (int64_t)blockIdx.x * nchunk * (kN * kN);
#ifdef WKV6_TIMING
    long long *dbg = reinterpret_cast<long long *>(ckpt + (int64_t)gridDim.x * nchunk * (kN * kN));
    int dbg_n = 0;
#endif

    if (wave < 4) {
        // ------------------------------ consumer ------------------------------
        const int q = wave, g = lane >> 4, l16 = lane & 15;
        const int col = 16 * q + l16;   // the channel this lane's accumulator column holds (j for gr/gk/gw, i for gv)
        int item = 0;
        if (kSweepStates) {
            // phase 1: S^T (rows i, column j = col), checkpoint at every chunk start
            f32x4 S[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) S[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
            for (int c = 0; c < nchunk; ++c, ++item) {
                __syncthreads();
                const BwdBuf &B = buf[item & 1];
                float *dst = ck + (int64_t)c * (kN * kN) + col * kN;
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    *reinterpret_cast<float4 *>(dst + 16 * m + 4 * g) = make_float4(S[m][0], S[m][1], S[m][2], S[m][3]);
                if (c + 1 == nchunk) break;   // the state after the last chunk is never used
#pragma unroll 1
                for (int p = 0; p < 4; ++p) {
                    if (c * CL + 16 * p >= T) break;
                    const s16x4 kq = frag_ct(B.ktT, col, 16 * p + 4 * g);
                    const float gq = B.g[p][col];
#pragma unroll
                    for (int m = 0; m < 4; ++m) S[m] = mfma16(frag_ct(B.vT, 16 * m + l16, 16 * p + 4 * g), kq, S[m]);
                    settle(S[0], S[1], S[2], S[3]);
#pragma unroll
                    for (int m = 0; m < 4; ++m) { S[m][0] *= gq; S[m][1] *= gq; S[m][2] *= gq; S[m][3] *= gq; }
                }
            }
            if (nchunk >= 1) ++item;   // account for the `break` above skipping the increment
        }
        // phase 2
        float (*vgyw)[16] = buf[0].vgyw;
        f32x4 Gj[4];   // reverse state, rows i, column j = col (the copy with rows j lives in waves 4..7)
#pragma unroll
        for (int m = 0; m < 4; ++m) Gj[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        const float uj = load1(u + h * kN + col);
        float gu_acc = 0.f;
        const bf16_t *rb = r + base, *kb_ = k + base, *vb = v + base, *wb = w + base, *gb = gy + base;   // uniform
        bf16_t *gr_h = gr + base, *gk_h = gk + base, *gw_h = gw + base;
        const uint32_t rowbytes = (uint32_t)C * 2u;
        // Software pipeline over the tiles: the gY / V fragments of the NEXT tile (possibly the top
        // tile of the next chunk) are requested as soon as the MFMAs of the current one have consumed
        // theirs, so that the epilogue covers their latency.  They land in their own registers and are
        // moved over at the top of the next iteration.  Rows past T are read from row T-1: they only
        // ever meet zero operands and are never stored.
        auto rowoff = [&](int t) { return (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes; };
        bf16x8 gf0, gf1, vf0, vf1, ngf0, ngf1, nvf0, nvf1;
        auto load_frags = [&](int tile_t0) {
            const uint32_t o = rowoff(tile_t0 + l16);
            ngf0 = frag_global(gb, o, 0, g); ngf1 = frag_global(gb, o, 1, g);
            nvf0 = frag_global(vb, o, 0, g); nvf1 = frag_global(vb, o, 1, g);
        };
        for (int c = nchunk - 1; c >= 0; --c, ++item) {
            // forward state at the chunk start, straight from the checkpoint (written by this same lane)
            f32x4 S[4];
            {
                const float *src = ck + (int64_t)c * (kN * kN) + col * kN;
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 x = *reinterpret_cast<const float4 *>(src + 16 * m + 4 * g);
                    S[m] = (f32x4){x.x, x.y, x.z, x.w};
                }
            }
            WKV6_STAMP();
            __syncthreads();
            WKV6_STAMP();
            const BwdBuf &B = buf[item & 1];
            const int t0 = c * CL;
            // states at the four tile starts as packed bf16 operands
            bf16x8 SopL[4], SopH[4];
            SopL[0] = acc_as_operand(S[0], S[1]); SopH[0] = acc_as_operand(S[2], S[3]);
#pragma unroll
            for (int p = 0; p < 3; ++p) {
                if (t0 + 16 * (p + 1) >= T) continue;   // uniform: no tile starts there
                const s16x4 kq = frag_ct(B.ktT, col, 16 * p + 4 * g);
                const float gq = B.g[p][col];
#pragma unroll
                for (int m = 0; m < 4; ++m) S[m] = mfma16(frag_ct(B.vT, 16 * m + l16, 16 * p + 4 * g), kq, S[m]);
                settle(S[0], S[1], S[2], S[3]);
#pragma unroll
                for (int m = 0; m < 4; ++m) { S[m][0] *= gq; S[m][1] *= gq; S[m][2] *= gq; S[m][3] *= gq; }
                SopL[p + 1] = acc_as_operand(S[0], S[1]); SopH[p + 1] = acc_as_operand(S[2], S[3]);
            }
            int ptop = 3;
            while (ptop > 0 && t0 + 16 * ptop >= T) --ptop;
            if (c == nchunk - 1) load_frags(t0 + 16 * ptop);   // later chunks: requested by the previous chunk's last tile
            WKV6_STAMP();
#pragma unroll
            for (int p = 3; p >= 0; --p) {
                if (p > ptop) continue;   // uniform: tiles past the end of the sequence
                gf0 = ngf0; gf1 = ngf1; vf0 = nvf0; vf1 = nvf1;
                const bf16x8 sL = SopL[p], sH = SopH[p];
                const int row = 16 * p + l16;           // tile-local token l16 as a chunk row
                const int tk = 16 * p + 4 * g;          // first of this lane group's 4 accumulator-row tokens
                // raw r, k, w of the accumulator rows (tokens tk..tk+3, channel col): used by the epilogue only
                float rraw[4], kraw[4], wraw[4];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const uint32_t o = rowoff(t0 + tk + rr) + 2u * (uint32_t)col;
                    rraw[rr] = bf16_bits_to_float(ld16(rb, o)); kraw[rr] = bf16_bits_to_float(ld16(kb_, o));
                    wraw[rr] = bf16_bits_to_float(ld16(wb, o));
                }
                const s16x4 rtq = frag_ct(B.rtT, col, tk), ktq = frag_ct(B.ktT, col, tk);
                // 16x16 intra-tile matrices
                f32x4 dA = {0.f, 0.f, 0.f, 0.f}, dAT = dA;
                dA = mfma32(gf0, vf0, dA);   dA = mfma32(gf1, vf1, dA);     // rows t, col s
                dAT = mfma32(vf0, gf0, dAT); dAT = mfma32(vf1, gf1, dAT);   // rows s, col t
                settle(dA, dAT);
                // the diagonal of dA is <v_t, gy_t>: lanes holding it publish it to this wave's LDS slot
                if ((l16 >> 2) == g) {
                    const int rs = l16 & 3;
                    vgyw[q][l16] = (rs == 0) ? dA[0] : (rs == 1) ? dA[1] : (rs == 2) ? dA[2] : dA[3];
                }
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int x = 4 * g + rr;
                    dA[rr] = (x > l16) ? dA[rr] : 0.f;
                    dAT[rr] = (l16 > x) ? dAT[rr] : 0.f;
                }
                // X (rows t, col j)
                f32x4 X = {0.f, 0.f, 0.f, 0.f};
                X = mfma16(pack4(dAT), ktq, X);
                chain_gap(X);
                X = mfma32(gf0, sL, X);
                X = mfma32(gf1, sH, X);
                // W (rows s, col j); Gj is decayed first so that W picks up g_j G
                const float gq = B.g[p][col];
#pragma unroll
                for (int m = 0; m < 4; ++m) { Gj[m][0] *= gq; Gj[m][1] *= gq; Gj[m][2] *= gq; Gj[m][3] *= gq; }
                f32x4 W = {0.f, 0.f, 0.f, 0.f};
                W = mfma16(pack4(dA), rtq, W);
                chain_gap(W);
                W = mfma32(vf0, acc_as_operand(Gj[0], Gj[1]), W);
                W = mfma32(vf1, acc_as_operand(Gj[2], Gj[3]), W);
                // next tile: p-1 of this chunk, else the top tile of the chunk before (always full),
                // else (very last tile of the sweep) this one again, unused
                load_frags(p > 0 ? t0 + 16 * (p - 1) : (c > 0 ? t0 - 16 : t0));
                // G <- diag(g) G + R~^T gY   (this wave's copy)
#pragma unroll
                for (int m = 0; m < 4; ++m) Gj[m] = mfma16(frag_ct(B.gyT, 16 * m + l16, tk), rtq, Gj[m]);
                settle(X, W, Gj);   // all read by VALU code from here on
                // tile-boundary term E[j] = sum_i S0[j][i] G_new[j][i]
                float E;
                {
                    float sl[8], sh[8], e0 = 0.f, e1 = 0.f, e2 = 0.f, e3 = 0.f;
                    unpack8(sL, sl); unpack8(sH, sh);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        e0 = fmaf(sl[e], Gj[0][e], e0); e1 = fmaf(sl[4 + e], Gj[1][e], e1);
                        e2 = fmaf(sh[e], Gj[2][e], e2); e3 = fmaf(sh[4 + e], Gj[3][e], e3);
                    }
                    E = (e0 + e1) + (e2 + e3);
                    E += __shfl_xor(E, 16);
                    E += __shfl_xor(E, 32);
                }
                // epilogue on the accumulator rows (tokens tk..tk+3, channel col)
                const float4 f4 = *reinterpret_cast<const float4 *>(&B.fr[col][20 * p + 4 * g]);
                const float f5 = B.fr[col][20 * p + 4 * g + 4];
                const float4 vg4 = *reinterpret_cast<const float4 *>(&vgyw[q][4 * g]);
                const float fr_[5] = {f4.x, f4.y, f4.z, f4.w, f5};
                float vg_[4] = {vg4.x, vg4.y, vg4.z, vg4.w};
                if (kRagged) {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) vg_[rr] = (t0 + tk + rr < T) ? vg_[rr] : 0.f;
                }
                float rt_[4], kt_[4], P[4], D[4], gro[4], gko[4];
                unpack4(rtq, rt_); unpack4(ktq, kt_);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    P[rr] = rt_[rr] * X[rr];
                    D[rr] = kt_[rr] * W[rr] - P[rr];
                    const float uvg = uj * vg_[rr];
                    gro[rr] = fmaf(fr_[rr], X[rr], uvg * kraw[rr]);
                    gko[rr] = fmaf(__builtin_amdgcn_rcpf(fr_[rr + 1]), W[rr], uvg * rraw[rr]);
                    gu_acc = fmaf(rraw[rr] * kraw[rr], vg_[rr], gu_acc);
                }
                // exclusive prefix of D over the 16 tokens: 4 in this lane, the rest in the lane groups below
                const float tot = D[0] + D[1] + D[2] + D[3];
                const float o1 = __shfl_up(tot, 16), o2 = __shfl_up(tot, 32), o3 = __shfl_up(tot, 48);
                float pre = E + ((g >= 1) ? o1 : 0.f) + ((g >= 2) ? o2 : 0.f) + ((g >= 3) ? o3 : 0.f);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int t = t0 + tk + rr;
                    const float ew = fast_exp(wraw[rr]);
                    // gw carries a factor exp(-ew): zero once that underflows (keeps exp(w) from
                    // amplifying rounding residue); first and last token are zero by definition
                    float gwv = (ew >= 88.f || t == 0 || t == T - 1) ? 0.f : -ew * (pre - P[rr]);
                    pre += D[rr];
                    if (!kRagged || t < T) {
                        const uint32_t o = (uint32_t)t * rowbytes + 2u * (uint32_t)col;
                        st16(gr_h, o, gro[rr]); st16(gk_h, o, gko[rr]); st16(gw_h, o, gwv);
                    }
                }
                WKV6_STAMP();
            }
        }
        // gu: fold the four lane groups (different tokens, same channel) with wavefront shuffles
        gu_acc += __shfl_xor(gu_acc, 16);
        gu_acc += __shfl_xor(gu_acc, 32);
        if (g == 0) store1(gu + (int64_t)b * C + h * kN + col, gu_acc);
    } else {
        // ------------------------------ producer ------------------------------
        const int p = wave - 4, ch = lane;
        const float uc = load1(u + h * kN + ch);
        const bf16_t *rb = r + base, *kb_ = k + base, *vb = v + base, *wb = w + base, *gb = gy + base;   // uniform
        const uint32_t rowbytes = (uint32_t)C * 2u;
        uint32_t qr[16], qk[16], qv[16], qw[16], qg[16];
        // item -> (chunk, full): phase 1 items need only k, v, w
        auto item_chunk = [&](int it) { return kSweepStates ? (it < nchunk ? it : 2 * nchunk - 1 - it) : nchunk - 1 - it; };
        auto item_full = [&](int it) { return kSweepStates ? it >= nchunk : true; };
        // Tokens past the end read as r = k = v = gy = 0, w = -inf (exp(w) = 0, decay 1).  Without
        // kRagged a tile is either entirely inside the sequence or entirely outside.
        auto prefetch = [&](int it) {
            const int tb = item_chunk(it) * CL + 16 * p;
            const bool full = item_full(it);
            if (tb < T) {   // uniform: a tile entirely past the end is neither loaded, prepared nor consumed
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int t = tb + e;
                    const bool ok = !kRagged || t < T;
                    const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + 2u * (uint32_t)ch;
                    const uint32_t bb = ld16(kb_, o), cc = ld16(vb, o), dd = ld16(wb, o);
                    qk[e] = ok ? bb : 0u; qv[e] = ok ? cc : 0u; qw[e] = ok ? dd : 0xff80u;
                }
                if (full) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int t = tb + e;
                        const bool ok = !kRagged || t < T;
                        const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + 2u * (uint32_t)ch;
                        const uint32_t a = ld16(rb, o), gg = ld16(gb, o);
                        qr[e] = ok ? a : 0u; qg[e] = ok ? gg : 0u;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e) { qr[e] = 0u; qg[e] = 0u; }
                }
            }
        };
        auto prepare = [&](int it) {
            BwdBuf &B = buf[it & 1];
            const bool full = item_full(it);
            const bool tile_in = item_chunk(it) * CL + 16 * p < T;
            float fr[16], fk[16], fw[16];
            uint32_t vbits[8], gbits[8];
            if (tile_in) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    fr[e] = bf16_bits_to_float(qr[e]); fk[e] = bf16_bits_to_float(qk[e]); fw[e] = bf16_bits_to_float(qw[e]);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    vbits[e] = qv[2 * e] | (qv[2 * e + 1] << 16);
                    gbits[e] = qg[2 * e] | (qg[2 * e + 1] << 16);
                }
            }
            if (it + 1 < nitem) prefetch(it + 1);
            if (tile_in) {

            // exponents are kept in base 2 (one v_exp_f32 each, no extra scaling multiply)
            float xr[16], xk[16], pr[16], fa[17];
            float cs2 = 0.f, pa = 1.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float ew2 = exp2_fast(fw[e] * kLog2e) * kLog2e;   // exp(w) * log2(e)
                fa[e] = pa;
                xr[e] = fr[e] * pa;
                cs2 += ew2;
                xk[e] = fk[e] * exp2_fast(cs2);
                pa *= exp2_fast(-ew2);
                pr[e] = fr[e] * uc * fk[e];
            }
            fa[16] = pa;
            if (__builtin_amdgcn_ballot_w64(!(cs2 <= kWildLimit * kLog2e)) != 0ull) {
                if (lane == 0) s_wild = 1;
            }
            uint32_t pk[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) pk[e] = pack_bf16x2(xk[2 * e], xk[2 * e + 1]);
            *reinterpret_cast<uint4 *>(&B.ktT[ch][16 * p]) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            *reinterpret_cast<uint4 *>(&B.ktT[ch][16 * p + 8]) = make_uint4(pk[4], pk[5], pk[6], pk[7]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p]) = make_uint4(vbits[0], vbits[1], vbits[2], vbits[3]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p + 8]) = make_uint4(vbits[4], vbits[5], vbits[6], vbits[7]);
            B.g[p][ch] = pa;
            if (full) {
                store_rows_paired(B.rt, 16 * p, lane, xr);
                store_rows_paired(B.kt, 16 * p, lane, xk);
#pragma unroll
                for (int e = 0; e < 8; ++e) pk[e] = pack_bf16x2(xr[2 * e], xr[2 * e + 1]);
                *reinterpret_cast<uint4 *>(&B.rtT[ch][16 * p]) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
                *reinterpret_cast<uint4 *>(&B.rtT[ch][16 * p + 8]) = make_uint4(pk[4], pk[5], pk[6], pk[7]);
                *reinterpret_cast<uint4 *>(&B.gyT[ch][16 * p]) = make_uint4(gbits[0], gbits[1], gbits[2], gbits[3]);
                *reinterpret_cast<uint4 *>(&B.gyT[ch][16 * p + 8]) = make_uint4(gbits[4], gbits[5], gbits[6], gbits[7]);
#pragma unroll
                for (int e = 0; e < 16; e += 4)
                    *reinterpret_cast<float4 *>(&B.fr[ch][20 * p + e]) = make_float4(fa[e], fa[e + 1], fa[e + 2], fa[e + 3]);
                B.fr[ch][20 * p + 16] = fa[16];
                const float tr = transpose_reduce16(pr, lane);
                if ((lane & 3) == 0) B.ruk[16 * p + ((lane >> 2) & 15)] = tr;
            }
            }
        };
        // gv role (second half of the consumer work, on the waves the operand preparation leaves
        // mostly idle): wave 4+q owns value columns i = 16q..16q+15 of the reverse state Gi (rows j).
        const int g = lane >> 4, l16 = lane & 15;
        const int col = 16 * p + l16;
        f32x4 Gi[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) Gi[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        bf16_t *gv_h = gv + base;
        auto gv_tiles = [&](int it) {
            const BwdBuf &B = buf[it & 1];
            const int t0 = item_chunk(it) * CL;
            int ptop = 3;
            while (ptop > 0 && t0 + 16 * ptop >= T) --ptop;
#pragma unroll 1
            for (int pp = ptop; pp >= 0; --pp) {
                const int row = 16 * pp + l16, tk = 16 * pp + 4 * g;
                const bf16x8 rf0 = frag_tc(B.rt, row, 0, g), rf1 = frag_tc(B.rt, row, 1, g);
                const bf16x8 kf0 = frag_tc(B.kt, row, 0, g), kf1 = frag_tc(B.kt, row, 1, g);
                const s16x4 gyq = frag_ct(B.gyT, col, tk);
                const float rukv = B.ruk[row];
                f32x4 A = {0.f, 0.f, 0.f, 0.f};
                A = mfma32(rf0, kf0, A); A = mfma32(rf1, kf1, A);   // rows t, col s
                settle(A);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int x = 4 * g + rr;
                    A[rr] = (x > l16) ? A[rr] : ((x == l16) ? rukv : 0.f);
                }
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 gg = *reinterpret_cast<const float4 *>(&B.g[pp][16 * m + 4 * g]);
                    Gi[m][0] *= gg.x; Gi[m][1] *= gg.y; Gi[m][2] *= gg.z; Gi[m][3] *= gg.w;
                }
                f32x4 GV = {0.f, 0.f, 0.f, 0.f};
                GV = mfma16(pack4(A), gyq, GV);
                chain_gap(GV);
                GV = mfma32(kf0, acc_as_operand(Gi[0], Gi[1]), GV);
                GV = mfma32(kf1, acc_as_operand(Gi[2], Gi[3]), GV);
#pragma unroll
                for (int m = 0; m < 4; ++m) Gi[m] = mfma16(frag_ct(B.rtT, 16 * m + l16, tk), gyq, Gi[m]);
                settle(GV, Gi);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int t = t0 + tk + rr;
                    if (!kRagged || t < T) st16(gv_h, (uint32_t)t * rowbytes + 2u * (uint32_t)col, GV[rr]);
                }
            }
        };
        prefetch(0);
        prepare(0);
        for (int it = 0; it < nitem; ++it) {
            WKV6_STAMP();
            __syncthreads();
            WKV6_STAMP();
            if (it + 1 < nitem) prepare(it + 1);
            WKV6_STAMP();
            if (item_full(it)) gv_tiles(it);
        }
    }
    // exact second pass for this (b, h) if any of its tiles left the representable range; the
    // workgroup's own slice of the state workspace (nchunk x 64 x 64 floats = T' x 64) holds P
    __threadfence_block();   // workgroup scope is enough (and a device-scope fence would write back the L2)
    __syncthreads();
    if (s_wild) {
        scan_bwd_a_body<bf16_t, bf16_t>(*reinterpret_cast<ScanBwdALds *>(smem), b, h, T, H, r, k, v, w, u, gy, gr, gu, ck, kN);
        __threadfence_block();
        __syncthreads();
        scan_bwd_b_body<bf16_t, bf16_t>(*reinterpret_cast<ScanBwdBLds *>(smem), b, h, T, H, r, k, v, w, u, gy, ck, kN, gk, gv, gw);
    }
}

size_t chunk_backward_workspace_bytes(int64_t B, int64_t T, int64_t H) {
    const int64_t nchunk = (T + CL - 1) / CL;
    return (size_t)(B * H * nchunk) * kN * kN * sizeof(float);
}

hipError_t chunk_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, bool states_ready)
{
    const size_t lds = 2 * sizeof(BwdBuf);
    auto launch = [&](auto kern) -> hipError_t {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(512), lds, st, (int)T, (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const bf16_t *)gy, (bf16_t *)gr, (bf16_t *)gk, (bf16_t *)gv, (bf16_t *)gw, (bf16_t *)gu,
                           (float *)workspace);
        return hipGetLastError();
    };
    const bool ragged = (T % 16) != 0;
    if (states_ready) return ragged ? launch(chunk_bwd_kernel<false, true>) : launch(chunk_bwd_kernel<false, false>);
    return ragged ? launch(chunk_bwd_kernel<true, true>) : launch(chunk_bwd_kernel<true, false>);
}

hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states)
{
    const size_t lds = 2 * sizeof(FwdBuf);
    auto launch = [&](auto kern, auto *state_tag) -> hipError_t {
        typedef std::remove_pointer_t<decltype(state_tag)> Ts;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(512), lds, st, (int)T, (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const Ts *)s0, map, (bf16_t *)y, (Ts *)sT, (float *)saved_states);
        return hipGetLastError();
    };
    const bool save = saved_states != nullptr, ragged = (T % 16) != 0;
    float *f32tag = nullptr;
    bf16_t *bf16tag = nullptr;
    if (state_dtype == kF32) {
        if (ragged) return save ? launch(chunk_fwd_kernel<float, true, true>, f32tag) : launch(chunk_fwd_kernel<float, false, true>, f32tag);
        return save ? launch(chunk_fwd_kernel<float, true, false>, f32tag) : launch(chunk_fwd_kernel<float, false, false>, f32tag);
    }
    if (ragged) return save ? launch(chunk_fwd_kernel<bf16_t, true, true>, bf16tag) : launch(chunk_fwd_kernel<bf16_t, false, true>, bf16tag);
    return save ? launch(chunk_fwd_kernel<bf16_t, true, false>, bf16tag) : launch(chunk_fwd_kernel<bf16_t, false, false>, bf16tag);
}

}  // namespace wkv6
