// WKV6 backward in chunk-parallel form for gfx950 (bf16 MFMA, fp32 states); the forward kernel and
// the notation are in wkv6_chunk_fwd.hip.
#include "wkv6_mfma.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>

namespace wkv6 {

constexpr int CL = 64;   // tokens per chunk
constexpr int LDT = 72;  // row pitch (elements) of [channel][token] operand arrays: 144 B, 16-byte aligned rows

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
        uint32_t nraw_r[4], nraw_k[4], nraw_w[4];   // raw r, k, w of the next tile's accumulator rows (epilogue only)
        auto load_frags = [&](int tile_t0) {
            const uint32_t o = rowoff(tile_t0 + l16);
            ngf0 = frag_global(gb, o, 0, g); ngf1 = frag_global(gb, o, 1, g);
            nvf0 = frag_global(vb, o, 0, g); nvf1 = frag_global(vb, o, 1, g);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const uint32_t oo = rowoff(tile_t0 + 4 * g + rr) + 2u * (uint32_t)col;
                nraw_r[rr] = ld16(rb, oo); nraw_k[rr] = ld16(kb_, oo); nraw_w[rr] = ld16(wb, oo);
            }
        };
        // checkpointed forward state of a chunk (written by this same lane in the forward pass)
        f32x4 S[4];
        auto load_state = [&](int c) {
            const float *src = ck + (int64_t)c * (kN * kN) + col * kN;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float4 x = *reinterpret_cast<const float4 *>(src + 16 * m + 4 * g);
                S[m] = (f32x4){x.x, x.y, x.z, x.w};
            }
        };
        if (!kSweepStates && nchunk > 0) load_state(nchunk - 1);
        for (int c = nchunk - 1; c >= 0; --c, ++item) {
            // with kSweepStates the checkpoints were written by this kernel a moment ago: read them
            // here; otherwise the load was issued during the previous chunk
            if (kSweepStates) load_state(c);
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
            if (!kSweepStates && c > 0) load_state(c - 1);   // S is free again: fetch the next chunk's state under this chunk's work
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
                uint32_t raw_r[4], raw_k[4], raw_w[4];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) { raw_r[rr] = nraw_r[rr]; raw_k[rr] = nraw_k[rr]; raw_w[rr] = nraw_w[rr]; }
                const s16x4 rtq = frag_ct(B.rtT, col, tk), ktq = frag_ct(B.ktT, col, tk);
                // 16x16 intra-tile matrices
                f32x4 dA = {0.f, 0.f, 0.f, 0.f}, dAT = dA;
                dA = mfma32(gf0, vf0, dA);   dA = mfma32(gf1, vf1, dA);     // rows t, col s
                dAT = mfma32(vf0, gf0, dAT); dAT = mfma32(vf1, gf1, dAT);   // rows s, col t
                settle(dA, dAT);
                WKV6_STAMP();
                // the diagonal of dA is <v_t, gy_t>: lanes holding it publish it to this wave's LDS slot
                {
                    const float d01 = (l16 & 1) ? dA[1] : dA[0], d23 = (l16 & 1) ? dA[3] : dA[2];
                    const float dv = (l16 & 2) ? d23 : d01;
                    if ((l16 >> 2) == g) vgyw[q][l16] = dv;
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
                WKV6_STAMP();
                // next tile: p-1 of this chunk, else the top tile of the chunk before (always full),
                // else (very last tile of the sweep) this one again, unused
                load_frags(p > 0 ? t0 + 16 * (p - 1) : (c > 0 ? t0 - 16 : t0));
                WKV6_STAMP();
                // G <- diag(g) G + R~^T gY   (this wave's copy)
#pragma unroll
                for (int m = 0; m < 4; ++m) Gj[m] = mfma16(frag_ct(B.gyT, 16 * m + l16, tk), rtq, Gj[m]);
                settle(X, W, Gj);   // all read by VALU code from here on
                WKV6_STAMP();
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
                    E = sum_rows((e0 + e1) + (e2 + e3));
                }
                WKV6_STAMP();
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
                    const float rraw = bf16_bits_to_float(raw_r[rr]), kraw = bf16_bits_to_float(raw_k[rr]);
                    gro[rr] = fmaf(fr_[rr], X[rr], uvg * kraw);
                    gko[rr] = fmaf(__builtin_amdgcn_rcpf(fr_[rr + 1]), W[rr], uvg * rraw);
                    gu_acc = fmaf(rraw * kraw, vg_[rr], gu_acc);
                }
                // exclusive prefix of D over the 16 tokens: 4 in this lane, the rest in the lane groups below
                float pre = E + prefix_rows(D[0] + D[1] + D[2] + D[3], g);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int t = t0 + tk + rr;
                    // exp(w) <= kWildLimit here (anything larger sends this (b, h) to the exact second pass)
                    const float ew = fast_exp(bf16_bits_to_float(raw_w[rr]));
                    const float gwv = -ew * (pre - P[rr]);
                    pre += D[rr];
                    if (!kRagged || t < T) {
                        const uint32_t o = (uint32_t)t * rowbytes + 2u * (uint32_t)col;
                        st16(gr_h, o, gro[rr]); st16(gk_h, o, gko[rr]); st16(gw_h, o, gwv);
                    }
                }
                WKV6_STAMP();
            }
        }
        // the gradient of the first and the last decay is zero by definition: overwrite what the
        // flow balance left there (rounding residue), after this wave's own stores have landed
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (g == 0 && T > 0) {
            st16(gw_h, 2u * (uint32_t)col, 0.f);
            st16(gw_h, (uint32_t)(T - 1) * rowbytes + 2u * (uint32_t)col, 0.f);
        }
        // gu: fold the four lane groups (different tokens, same channel)
        gu_acc = sum_rows(gu_acc);
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
            WKV6_STAMP();
            if (it + 1 < nitem) prefetch(it + 1);
            WKV6_STAMP();
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
            WKV6_STAMP();
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

}  // namespace wkv6
