// WKV6 in chunk-parallel form for gfx950: bf16 MFMA for the dense products, fp32 state.
//
// One workgroup (8 waves) per (batch, head).  Time is cut into chunks of 64 tokens, each chunk
// into 4 tiles of 16 tokens.  The fp32 state S[j][i] lives in the MFMA accumulators of the four
// "consumer" waves (wave q owns value columns 16q..16q+15) and is advanced one tile at a time:
//
//   c_t = sum_{s<t} exp(w_s) inside the tile (so exp(-c_t) is the decay from the tile start to t)
//   R~[t][j] = r_t[j] exp(-c_t[j])            K~[t][j] = k_t[j] exp(+c_{t+1}[j])
//   g[j] = exp(-c_16[j])
//   A[t][s]  = R~_t . K~_s  (s < t),  A[t][t] = sum_j r_t[j] u[j] k_t[j]
//   Y        = R~ S + A V          (16x64x64 and 16x16x16 MFMA, K index j resp. s)
//   S       <- diag(g) (S + K~^T V)   (64x16x16 MFMA, K index s)
//
// Data path.  The raw r, k, w, v rows of a chunk go from global memory straight into LDS tiles
// (16-byte pieces, no registers), two chunks ahead of their use.  The four "producer" waves (wave
// 4+p prepares tile p, lane = channel) read r, k, w from there, compute R~, K~, g and the diagonal
// in fp32 for the NEXT chunk and write them back as bf16 tiles while the consumers run the MFMAs of
// the current one; the consumers take V directly from its raw tile.  Every tile is stored once,
// [token][channel]; fragments with the k-slots along the tokens come from the transposing LDS read.
// The two roles meet at one barrier per chunk.  HBM traffic is exactly the algorithmic minimum
// (r,k,v,w read once, y written once).
//
// exp(+c) needs the decay accumulated inside one 16-token tile to stay in range.  A producer wave
// that meets a tile whose summed exp(w) exceeds kWildLimit in any channel raises a flag in LDS, and
// the workgroup then redoes ITS (batch, head) pair with the exact per-timestep code
// (wkv6_scan_body.h) before the kernel ends; other workgroups are unaffected.
#include "wkv6_mfma.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>

namespace wkv6 {

constexpr int CL = 64;   // tokens per chunk

// LDS map of the forward kernel (byte offsets into the dynamic block)
struct FwdLds {
    static constexpr int kRawRKW = 0;                                   // [2 chunk parities][r,k,w] raw tiles
    static constexpr int kRawV = kRawRKW + 2 * 3 * kTileBytes;          // [3] raw v tiles (chunk % 3)
    static constexpr int kOp = kRawV + 3 * kTileBytes;                  // [2] operand blocks
    static constexpr int kOpRt = 0, kOpKt = kTileBytes, kOpG = 2 * kTileBytes, kOpRuk = kOpG + 4 * kN * 4;
    static constexpr int kOpBytes = kOpRuk + CL * 4;
    static constexpr int kBytes = kOp + 2 * kOpBytes;
};

// kSave: also write the state at every chunk start to `ckpt` (bf16, [b][h][chunk][j][i]) for the
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
    static_assert(sizeof(ScanFwdLds) <= FwdLds::kBytes, "the exact second pass reuses the LDS block");
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
                // bf16 [chunk][j][i], in the first half of this workgroup's slice of the workspace
                bf16_t *dst = reinterpret_cast<bf16_t *>(ckpt + (int64_t)blockIdx.x * nchunk * (kN * kN)) + (int64_t)c * (kN * kN) + 16 * q + l16;
#pragma unroll
                for (int m = 0; m < 4; ++m)
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) store1(dst + (16 * m + 4 * g + rr) * kN, S[m][rr]);
            }
            __syncthreads();
            const unsigned char *op = smem + FwdLds::kOp + (c & 1) * FwdLds::kOpBytes;
            const unsigned char *rt = op + FwdLds::kOpRt, *kt = op + FwdLds::kOpKt;
            const float *gv_ = reinterpret_cast<const float *>(op + FwdLds::kOpG);
            const float *ruk = reinterpret_cast<const float *>(op + FwdLds::kOpRuk);
            const unsigned char *vt = smem + FwdLds::kRawV + (c % 3) * kTileBytes;
            const int t0 = c * CL;
#pragma unroll 1
            for (int p = 0; p < 4; ++p) {
                if (t0 + 16 * p >= T) break;
                const int row = 16 * p + l16;
                const bf16x8 rf0 = tile_frag_ch(rt, row, 0, g), rf1 = tile_frag_ch(rt, row, 1, g);
                const bf16x8 kf0 = tile_frag_ch(kt, row, 0, g), kf1 = tile_frag_ch(kt, row, 1, g);
                const s16x4 vf = tile_frag_tok(vt, 16 * q, 16 * p, l16, g);
                const float rukv = ruk[row];
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
                for (int m = 0; m < 4; ++m) S[m] = mfma16(tile_frag_tok(kt, 16 * m, 16 * p, l16, g), vf, S[m]);
                settle(Y, S[0], S[1], S[2], S[3]);   // Y is stored, S scaled and converted by VALU code from here on
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 gg = *reinterpret_cast<const float4 *>(&gv_[p * kN + 16 * m + 4 * g]);
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
        // ------------------------------ producer: loads and operand preparation ------------------------------
        const int p = wave - 4, ch = lane;
        const float uc = load1(u + h * kN + ch);
        const bf16_t *rb = r + base, *kb_ = k + base, *vb = v + base, *wb = w + base;   // uniform
        const uint32_t rowbytes = (uint32_t)C * 2u;
        const uint32_t lds0 = lds_address(smem);
        // this lane's part of an 8-row block load: row (lane >> 3), 16-byte piece swizzled with the row
        const int lrow = lane >> 3;
        const uint32_t lpiece = (uint32_t)(((lane & 7) ^ lrow) << 4);
        // Rows past the end of the sequence are fetched from row T-1 (valid memory); the operand
        // preparation turns them into r = k = 0, w = -inf, and v rows that only ever meet zero
        // operands.  A tile entirely past the end is neither loaded, prepared nor consumed.
        auto issue_loads = [&](int c) -> bool {
            const int tb = c * CL + 16 * p;
            if (tb >= T) return false;
            const uint32_t rkw = lds0 + FwdLds::kRawRKW + (c & 1) * 3 * kTileBytes + 16 * p * kTileRow;
            const uint32_t vv = lds0 + FwdLds::kRawV + (c % 3) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int t = tb + 8 * hf + lrow;
                const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + lpiece;
                load_rows8_to_lds(rb, o, rkw + 8 * hf * kTileRow);
                load_rows8_to_lds(kb_, o, rkw + kTileBytes + 8 * hf * kTileRow);
                load_rows8_to_lds(wb, o, rkw + 2 * kTileBytes + 8 * hf * kTileRow);
                load_rows8_to_lds(vb, o, vv + 8 * hf * kTileRow);
            }
            return true;
        };
        // per-lane byte offsets of channel `ch` inside a tile row, for the 8 swizzle phases
        uint32_t choff[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) choff[s] = (uint32_t)((((ch >> 3) ^ s) << 4) + ((ch & 7) << 1)) + (uint32_t)(16 * p * kTileRow);
        auto prepare = [&](int c) {
            if (c * CL + 16 * p >= T) return;
            const unsigned char *raw = smem + FwdLds::kRawRKW + (c & 1) * 3 * kTileBytes;
            unsigned char *op = smem + FwdLds::kOp + (c & 1) * FwdLds::kOpBytes;
            float fr[16], fk[16], fw[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t o = choff[e & 7] + e * kTileRow;
                uint32_t a = *reinterpret_cast<const uint16_t *>(raw + o);
                uint32_t bb = *reinterpret_cast<const uint16_t *>(raw + kTileBytes + o);
                uint32_t dd = *reinterpret_cast<const uint16_t *>(raw + 2 * kTileBytes + o);
                if (kRagged && c * CL + 16 * p + e >= T) { a = 0u; bb = 0u; dd = 0xff80u; }
                fr[e] = bf16_bits_to_float(a); fk[e] = bf16_bits_to_float(bb); fw[e] = bf16_bits_to_float(dd);
            }
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
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const uint32_t pr2 = pack_bf16x2(xr[e], xr[e + 1]), pk2 = pack_bf16x2(xk[e], xk[e + 1]);
                const uint32_t o0 = choff[e & 7] + e * kTileRow, o1 = choff[(e + 1) & 7] + (e + 1) * kTileRow;
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpRt + o0) = (uint16_t)pr2;
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpRt + o1) = (uint16_t)(pr2 >> 16);
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpKt + o0) = (uint16_t)pk2;
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpKt + o1) = (uint16_t)(pk2 >> 16);
            }
            reinterpret_cast<float *>(op + FwdLds::kOpG)[p * kN + ch] = pa;
            const float tot = transpose_reduce16(pr, lane);
            if ((lane & 3) == 0) reinterpret_cast<float *>(op + FwdLds::kOpRuk)[16 * p + ((lane >> 2) & 15)] = tot;
        };
        // chunk c is loaded during iteration c-2 (or the prologue), prepared during iteration c-1
        issue_loads(0);
        bool next_in_flight = nchunk > 1 && issue_loads(1);
        if (next_in_flight) wait_loads<8>(); else wait_loads<0>();
        prepare(0);
        for (int c = 0; c < nchunk; ++c) {
            __syncthreads();
            // the raw r, k, w block of chunk c (read by this wave's prepare(c) before the barrier) and the
            // raw v block of chunk c-1 (read by the consumers before the barrier) are free again
            const bool far_in_flight = c + 2 < nchunk && issue_loads(c + 2);
            if (c + 1 < nchunk) {
                if (far_in_flight) wait_loads<8>(); else wait_loads<0>();
                prepare(c + 1);
            }
        }
        wait_loads<0>();
    }
    // exact second pass for this (b, h) if any of its tiles left the representable range
    __threadfence_block();   // workgroup scope is enough (and a device-scope fence would write back the L2)
    __syncthreads();
    if (s_wild)
        scan_fwd_body<bf16_t, bf16_t, Ts>(*reinterpret_cast<ScanFwdLds *>(smem), b, h, T, H, r, k, v, w, u, s0, map, y, sT);
}

hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states)
{
    const size_t lds = FwdLds::kBytes;
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
