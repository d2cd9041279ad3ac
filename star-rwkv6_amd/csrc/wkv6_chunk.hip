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
// exp(+c) needs the decay accumulated inside one 16-token tile to stay in range.  A tile whose
// summed exp(w) exceeds kWildLimit in any channel raises a flag; the launcher always enqueues the
// exact per-timestep kernel behind this one, and that kernel runs only if the flag was raised.
#include "wkv6_common.h"
#include "wkv6_kernels.h"

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
__device__ __forceinline__ float xor1(float x) {   // value of the neighbouring lane (lane ^ 1)
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));
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
    uint16_t kbT[kN][LDT];  // K^[t][j] stored [j][t]
    uint16_t vT[kN][LDT];   // V[t][i]  stored [i][t]
    float g[4][kN];         // per-tile decay exp(-c_16)
    float ruk[CL];          // sum_j r u k per token
};

template <typename Ts>
__global__ __launch_bounds__(512) void chunk_fwd_kernel(int T, int H,
        const bf16_t *__restrict__ r, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v,
        const bf16_t *__restrict__ w, const bf16_t *__restrict__ u,
        const Ts *__restrict__ s0, const int64_t *__restrict__ map,
        bf16_t *__restrict__ y, Ts *__restrict__ sT,
        unsigned long long *__restrict__ wild_flag, unsigned long long epoch)
{
    extern __shared__ __align__(16) unsigned char smem[];
    FwdBuf *buf = reinterpret_cast<FwdBuf *>(smem);

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
        for (int c = 0; c < nchunk; ++c) {
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
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int s = 4 * g + rr;
                    AT[rr] = (l16 > s) ? AT[rr] : ((l16 == s) ? rukv : 0.f);
                }
                // Y += A V : the masked A^T accumulator IS the A operand (row t = l16, k-slots s = 4g+r)
                Y = mfma16(make_s16x4(pack_bf16x2(AT[0], AT[1]), pack_bf16x2(AT[2], AT[3])), vf, Y);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int t = t0 + 16 * p + 4 * g + rr;
                    if (t < T) store1(y + base + (int64_t)t * C + 16 * q + l16, Y[rr]);
                }
                // S <- diag(g) S + K^T V
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 gg = *reinterpret_cast<const float4 *>(&B.g[p][16 * m + 4 * g]);
                    S[m][0] *= gg.x; S[m][1] *= gg.y; S[m][2] *= gg.z; S[m][3] *= gg.w;
                    S[m] = mfma16(frag_ct(B.kbT, 16 * m + l16, 16 * p + 4 * g), vf, S[m]);
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
        const uint16_t *r16 = reinterpret_cast<const uint16_t *>(r) + base + ch;
        const uint16_t *k16 = reinterpret_cast<const uint16_t *>(k) + base + ch;
        const uint16_t *v16 = reinterpret_cast<const uint16_t *>(v) + base + ch;
        const uint16_t *w16 = reinterpret_cast<const uint16_t *>(w) + base + ch;
        uint32_t qr[16], qk[16], qv[16], qw[16];
        auto prefetch = [&](int c) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int t = c * CL + 16 * p + e;
                if (t < T) {
                    const int64_t o = (int64_t)t * C;
                    qr[e] = r16[o]; qk[e] = k16[o]; qv[e] = v16[o]; qw[e] = w16[o];
                } else {
                    qr[e] = 0; qk[e] = 0; qv[e] = 0; qw[e] = 0xff80u;  // w = -inf: exp(w) = 0, decay 1
                }
            }
        };
        auto prepare = [&](int c) {   // consumes the prefetched registers, refills them for chunk c+1
            FwdBuf &B = buf[c & 1];
            float fr[16], fk[16], fw[16];
            uint32_t vbits[8];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                fr[e] = bf16_bits_to_float(qr[e]); fk[e] = bf16_bits_to_float(qk[e]); fw[e] = bf16_bits_to_float(qw[e]);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) vbits[e] = qv[2 * e] | (qv[2 * e + 1] << 16);
            if (c + 1 < nchunk) prefetch(c + 1);

            float d[16], xr[16], xk[16], pr[16];
            float cs = 0.f, pa = 1.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float ew = fast_exp(fw[e]);
                d[e] = fast_exp(-ew);
                xr[e] = fr[e] * pa;          // r exp(-c_t)
                cs += ew;
                xk[e] = fk[e] * fast_exp(cs);  // k exp(+c_{t+1})
                pa *= d[e];
                pr[e] = fr[e] * uc * fk[e];
            }
            if (__builtin_amdgcn_ballot_w64(!(cs <= kWildLimit)) != 0ull) {
                if (lane == 0 && wild_flag != nullptr) *wild_flag = epoch;
            }
            store_rows_paired(B.rt, 16 * p, lane, xr);
            store_rows_paired(B.kt, 16 * p, lane, xk);
            float pb = 1.f;
#pragma unroll
            for (int e = 15; e >= 0; --e) { xk[e] = fk[e] * pb; pb *= d[e]; }   // k exp(-(c_16 - c_{t+1}))
            uint32_t kb[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) kb[e] = pack_bf16x2(xk[2 * e], xk[2 * e + 1]);
            *reinterpret_cast<uint4 *>(&B.kbT[ch][16 * p]) = make_uint4(kb[0], kb[1], kb[2], kb[3]);
            *reinterpret_cast<uint4 *>(&B.kbT[ch][16 * p + 8]) = make_uint4(kb[4], kb[5], kb[6], kb[7]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p]) = make_uint4(vbits[0], vbits[1], vbits[2], vbits[3]);
            *reinterpret_cast<uint4 *>(&B.vT[ch][16 * p + 8]) = make_uint4(vbits[4], vbits[5], vbits[6], vbits[7]);
            B.g[p][ch] = pa;
            const float tot = transpose_reduce16(pr, lane);
            if ((lane & 3) == 0) B.ruk[16 * p + ((lane >> 2) & 15)] = tot;
        };
        prefetch(0);
        prepare(0);
        for (int c = 0; c < nchunk; ++c) {
            __syncthreads();
            if (c + 1 < nchunk) prepare(c + 1);
        }
    }
}

hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT,
                         unsigned long long *wild_flag, unsigned long long epoch)
{
    const size_t lds = 2 * sizeof(FwdBuf);
    hipError_t e;
    if (state_dtype == kF32) {
        auto kern = chunk_fwd_kernel<float>;
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(512), lds, st, (int)T, (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const float *)s0, map, (bf16_t *)y, (float *)sT, wild_flag, epoch);
    } else {
        auto kern = chunk_fwd_kernel<bf16_t>;
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(512), lds, st, (int)T, (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const bf16_t *)s0, map, (bf16_t *)y, (bf16_t *)sT, wild_flag, epoch);
    }
    return hipGetLastError();
}

}  // namespace wkv6
