// WKV6 backward in chunk-parallel form for gfx950 (bf16 MFMA, fp32 states); the forward kernel and
// the notation are in wkv6_chunk_fwd.hip.
//
// The forward state at every chunk start comes from the workspace (bf16, transposed: [b][h][chunk][i][j]), left
// there by the saving forward pass -- or, when the caller has none, by a state-only pass of the
// forward kernel that chunk_backward() runs first.  The kernel sweeps the chunks in reverse order
// with the reverse state G in MFMA accumulators.  G is kept twice, once with rows j / columns i (for gv) and once transposed (for
// gk), so that it can be fed back to the MFMAs as an operand without leaving the registers; the
// forward state at the tile starts of a chunk is recomputed from the checkpoint and held as packed
// bf16 operands.
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
//
// Workgroup: one per (batch, head).  (With more pairs than half the compute units the block-form
// kernel in wkv6_block_bwd.hip runs instead, unless gradients flow through the state or the tensors
// are fp16.)
// 12 waves in four-wave roles (one wave of each role per SIMD):
//   loader/producer (wave p <-> tile p, lane = channel): brings the raw r, k, w, v, gy rows of a
//       chunk from global memory straight into LDS tiles two items ahead (and the chunk's saved
//       forward state one item ahead), and one item ahead turns r, k, w into the bf16 tiles R~, K~
//       (written over the raw r, k), exp(-c_t) plus g and the diagonal sum r u k; the same
//       waves then run the gv role (wave q <-> value columns 16q..): reverse state with rows j,
//       produces gv;
//   two consumer groups (wave q <-> key columns 16q..): reverse state with rows i, produce gr, gk,
//       gw, gu.  Both groups advance G through every tile (4 MFMAs and a scaling) but share out the
//       expensive per-tile work: group 0 takes tiles 3 and 1, group 1 tiles 2 and 0.
// All tiles are stored once, [token][channel]; v and gy are consumed as they came from memory.
#include "wkv6_mfma.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>


namespace wkv6 {

constexpr int CL = 64;   // tokens per chunk


// LDS map of the backward kernel (byte offsets into the dynamic block); "item" = one chunk visit
struct BwdLds {
    static constexpr int kRawRK = 0;                                   // [item % 3][r, k] raw tiles, turned into R~, K~ in place
    static constexpr int kRawW = kRawRK + 3 * 2 * kTileBytes;          // [item % 3] raw w tiles
    static constexpr int kRawVG = kRawW + 3 * kTileBytes;              // [item % 3][v, gy] raw tiles
    static constexpr int kOp = kRawVG + 3 * 2 * kTileBytes;            // [item & 1] operand blocks
    static constexpr int kOpFr = 0;                                               // exp(-c_t) tile
    static constexpr int kOpG = kTileBytes, kOpRuk = kOpG + 4 * kN * 4;           // g[4][64], ruk[64] (fp32)
    static constexpr int kOpBytes = kOpRuk + CL * 4;
    static constexpr int kState = kOp + 2 * kOpBytes;                  // [item & 1] saved forward state of the chunk, bf16 [i][j] (transposed) as a tile
    static constexpr int kVgy = kState + 2 * kTileBytes;                    // [8 consumer waves][16] fp32: <v_t, gy_t>
    static constexpr int kGu = kVgy + 8 * 16 * 4;                      // [64] fp32: gu partial of consumer group 1
    static constexpr int kBytes = kGu + kN * 4;
};
static_assert(BwdLds::kBytes <= 160 * 1024, "LDS block of the backward kernel");

struct BwdArgs {
    int T, H;
    const bf16_t *r, *k, *v, *w, *u, *gy;   // 16-bit elements: bf16, or fp16 with v and gy bf16 copies (see OutOf)
    const void *v_orig, *gy_orig;           // v and gy as the caller holds them (read by the exact per-timestep pass)
    bf16_t *gr, *gk, *gv, *gw, *gu;         // elements of the output type (bf16, or fp32 for fp16 tensors)
    bf16_t *gu_sum;   // null, or C elements: receives the sum of gu over the batch
    int *arrivals;    // per head: workgroups that have delivered their gu partial (zero on entry)
    int B;
    float *ckpt;
    // gradients through the state (all null for the stateless operator): fp32 (B,H,64,64) [key][value]
    const float *s0, *gsT;   // initial state; gradient arriving at the final state
    float *gs0;              // receives dL/dS_0
};

// ------------------------------------------------------------------------------------------
// Consumer group GRP of two: gr, gk, gw, gu.
// ------------------------------------------------------------------------------------------
template <typename Tin, bool kRagged, int GRP>
__device__ __forceinline__ void bwd_consumer(const BwdArgs &a, unsigned char *smem, const int *s_wild, int pair0, int q, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int col = 16 * q + l16;   // the key channel j this lane's accumulator column holds
    const int64_t C = (int64_t)H * kN;
    const int h = pair0 % H, b = pair0 / H;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
    const int nchunk = (T + CL - 1) / CL;
    auto mine = [](int p) { return (p & 1) == (GRP ^ 1); };   // group 0: tiles 3, 1; group 1: tiles 2, 0
    int item = 0;
    float *vgyw = reinterpret_cast<float *>(smem + BwdLds::kVgy) + (4 * GRP + q) * 16;
    f32x4 Gj[4];   // reverse state, rows i, column j = col (the copy with rows j lives in the gv waves)
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        Gj[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (a.gsT) Gj[m] = *reinterpret_cast<const f32x4 *>(a.gsT + (int64_t)(b * H + h) * (kN * kN) + col * kN + 16 * m + 4 * g);
    }
    typedef typename OutOf<Tin>::type Tout;
    const float uj = load1(reinterpret_cast<const Tin *>(a.u) + h * kN + col);
    float gu_acc = 0.f;
    Tout *gr_h = reinterpret_cast<Tout *>(a.gr) + base, *gk_h = reinterpret_cast<Tout *>(a.gk) + base, *gw_h = reinterpret_cast<Tout *>(a.gw) + base;
    const uint32_t rowbytes = (uint32_t)C * (uint32_t)sizeof(Tout);
    float *gu_lds = reinterpret_cast<float *>(smem + BwdLds::kGu);
    // Saved forward state of a chunk as packed bf16: Sraw[m] = S^T[i = 16m + 4g .. +3][j = col].  It
    // comes out of LDS, where the producer waves put the chunk's block from the workspace.  The
    // consumer waves issue no global load at all:
    // their loads would queue behind their own gradient stores, and a wave's memory operations
    // complete in program order.
    uint2 Sraw[4];
    // One chunk visit.  All four tiles are always processed (tokens past the end were prepared as
    // r = k = 0, decay 1, so they leave both states alone and contribute nothing).
    // gr, gk, gw of the 4 tokens from `tfirst` on, channel col (bf16 outputs: two tokens share one conversion per tensor)
    auto store_tile = [&](int tfirst, const float (&gro)[4], const float (&gko)[4], const float (&gwo)[4]) {
        if constexpr (sizeof(Tout) == 2) {
            const uint32_t pk[6] = {pack_bf16x2(gro[0], gro[1]), pack_bf16x2(gko[0], gko[1]), pack_bf16x2(gwo[0], gwo[1]),
                                    pack_bf16x2(gro[2], gro[3]), pack_bf16x2(gko[2], gko[3]), pack_bf16x2(gwo[2], gwo[3])};
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int t = tfirst + 2 * hh;
                const uint32_t o = (uint32_t)t * rowbytes + 2u * (uint32_t)col;
                if (!kRagged || t < T) {
                    st16_lo(gr_h, o, pk[3 * hh]); st16_lo(gk_h, o, pk[3 * hh + 1]); st16_lo(gw_h, o, pk[3 * hh + 2]);
                }
                if (!kRagged || t + 1 < T) {
                    st16_hi(gr_h, o + rowbytes, pk[3 * hh]); st16_hi(gk_h, o + rowbytes, pk[3 * hh + 1]); st16_hi(gw_h, o + rowbytes, pk[3 * hh + 2]);
                }
            }
        } else {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int t = tfirst + rr;
                const uint32_t o = (uint32_t)t * rowbytes + 4u * (uint32_t)col;
                if (!kRagged || t < T) {
                    *reinterpret_cast<float *>(reinterpret_cast<char *>(gr_h) + o) = gro[rr];
                    *reinterpret_cast<float *>(reinterpret_cast<char *>(gk_h) + o) = gko[rr];
                    *reinterpret_cast<float *>(reinterpret_cast<char *>(gw_h) + o) = gwo[rr];
                }
            }
        }
    };
    auto visit = [&](int c, uint2 (&Sraw)[4]) {
        __syncthreads();
        {
            // the tile holds the state transposed (rows i, channels j): S^T[16m + 4g + e][col], e < 4, per read
            const unsigned char *stt = smem + BwdLds::kState + (item & 1) * kTileBytes;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const u32x2 x = __builtin_bit_cast(u32x2, tile_frag_tok(stt, 16 * q, 16 * m, l16, g));
                Sraw[m] = make_uint2(x[0], x[1]);
            }
        }
        // Uniform block offsets of this item.  They pass through fresh_s() before every tile, which
        // keeps the compiler from forming (block + lane offset) for all tiles at once and holding
        // two dozen address registers across the chunk.
        int op_off = BwdLds::kOp + (item & 1) * BwdLds::kOpBytes;
        int rk_off = BwdLds::kRawRK + (item % 3) * 2 * kTileBytes;
        int vg_off = BwdLds::kRawVG + (item % 3) * 2 * kTileBytes;
        int w_off = BwdLds::kRawW + (item % 3) * kTileBytes;
        const unsigned char *rt, *kt, *fr, *vt, *gyt, *wt;
        const float *gg;
        auto fresh_pointers = [&]() {
            op_off = fresh_s(op_off); vg_off = fresh_s(vg_off); w_off = fresh_s(w_off);
            rk_off = fresh_s(rk_off);
            rt = smem + rk_off; kt = smem + rk_off + kTileBytes; fr = smem + op_off + BwdLds::kOpFr;
            gg = reinterpret_cast<const float *>(smem + op_off + BwdLds::kOpG);
            vt = smem + vg_off; gyt = vt + kTileBytes; wt = smem + w_off;
        };
        fresh_pointers();
        const int t0 = c * CL;
        // states at the tile starts this group works on, as packed bf16 operands
        bf16x8 SopL[4], SopH[4];
        f32x4 S[4];
#pragma unroll
        for (int m = 0; m < 4; ++m)
            S[m] = (f32x4){__uint_as_float(Sraw[m].x << 16), __uint_as_float(Sraw[m].x & 0xffff0000u),
                           __uint_as_float(Sraw[m].y << 16), __uint_as_float(Sraw[m].y & 0xffff0000u)};
        if (mine(0)) {
            SopL[0] = make_bf16x8(Sraw[0].x, Sraw[0].y, Sraw[1].x, Sraw[1].y);
            SopH[0] = make_bf16x8(Sraw[2].x, Sraw[2].y, Sraw[3].x, Sraw[3].y);
        }
#pragma unroll
        for (int p = 0; p < 3; ++p) {
            if (GRP == 1 && p == 2) continue;   // group 1 needs the states of tiles 0 and 2 only
            const s16x4 kq = tile_frag_tok(kt, 16 * q, 16 * p, l16, g);
            const float gq = gg[p * kN + col];
#pragma unroll
            for (int m = 0; m < 4; ++m) S[m] = mfma16(tile_frag_tok(vt, 16 * m, 16 * p, l16, g), kq, S[m]);
            settle(S[0], S[1], S[2], S[3]);
#pragma unroll
            for (int m = 0; m < 4; ++m) { S[m][0] *= gq; S[m][1] *= gq; S[m][2] *= gq; S[m][3] *= gq; }
            if (mine(p + 1)) { SopL[p + 1] = acc_as_operand(S[0], S[1]); SopH[p + 1] = acc_as_operand(S[2], S[3]); }
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the scheduler from interleaving the tiles (register pressure)
#pragma unroll
        for (int p = 3; p >= 0; --p) {
            fresh_pointers();
            const float gq = gg[p * kN + col];
            const s16x4 rtq = tile_frag_tok(rt, 16 * q, 16 * p, l16, g);
            if (!mine(p)) {
                // the other group does this tile; only carry the reverse state across it
                f32x4 Upd[4];   // R~^T gY, off the chain through G
#pragma unroll
                for (int m = 0; m < 4; ++m) Upd[m] = mfma16(tile_frag_tok(gyt, 16 * m, 16 * p, l16, g), rtq, (f32x4){0.f, 0.f, 0.f, 0.f});
                settle(Upd[0], Upd[1], Upd[2], Upd[3]);
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    Gj[m][0] = fmaf(Gj[m][0], gq, Upd[m][0]); Gj[m][1] = fmaf(Gj[m][1], gq, Upd[m][1]);
                    Gj[m][2] = fmaf(Gj[m][2], gq, Upd[m][2]); Gj[m][3] = fmaf(Gj[m][3], gq, Upd[m][3]);
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            const bf16x8 sL = SopL[p], sH = SopH[p];
            const int row = 16 * p + l16;           // tile-local token l16 as a chunk row
            const int tk = 16 * p + 4 * g;          // first of this lane group's 4 accumulator-row tokens
            const bf16x8 gf0 = tile_frag_ch(gyt, row, 0, g), gf1 = tile_frag_ch(gyt, row, 1, g);
            const bf16x8 vf0 = tile_frag_ch(vt, row, 0, g), vf1 = tile_frag_ch(vt, row, 1, g);
            const s16x4 ktq = tile_frag_tok(kt, 16 * q, 16 * p, l16, g);
            // 16x16 intra-tile matrices
            f32x4 dA = {0.f, 0.f, 0.f, 0.f}, dAT = dA;
            dA = mfma32(gf0, vf0, dA);   dA = mfma32(gf1, vf1, dA);     // rows t, col s
            dAT = mfma32(vf0, gf0, dAT); dAT = mfma32(vf1, gf1, dAT);   // rows s, col t
            settle(dA, dAT);
            // the diagonal of dA is <v_t, gy_t>: lanes holding it publish it to this wave's LDS slot
            {
                const float d01 = (l16 & 1) ? dA[1] : dA[0], d23 = (l16 & 1) ? dA[3] : dA[2];
                const float dv = (l16 & 2) ? d23 : d01;
                if ((l16 >> 2) == g) vgyw[l16] = dv;
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
#pragma unroll
            for (int m = 0; m < 4; ++m) { Gj[m][0] *= gq; Gj[m][1] *= gq; Gj[m][2] *= gq; Gj[m][3] *= gq; }
            f32x4 W = {0.f, 0.f, 0.f, 0.f};
            W = mfma16(pack4(dA), rtq, W);
            chain_gap(W);
            W = mfma32(vf0, acc_as_operand(Gj[0], Gj[1]), W);
            W = mfma32(vf1, acc_as_operand(Gj[2], Gj[3]), W);
            // G <- diag(g) G + R~^T gY   (this wave's copy)
#pragma unroll
            for (int m = 0; m < 4; ++m) Gj[m] = mfma16(tile_frag_tok(gyt, 16 * m, 16 * p, l16, g), rtq, Gj[m]);
            settle(X, W, Gj);   // all read by VALU code from here on
            __builtin_amdgcn_sched_barrier(0);
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
            // epilogue on the accumulator rows (tokens tk..tk+3, channel col).  From the tiles:
            // a_t = exp(-c_t), R~ = r a_t, K~ = k / a_{t+1}, raw w; r and k themselves follow from these.
            float a_[5], w_[4], rt_[4], kt_[4];
            {
                float a4[4], nx[4];
                unpack4(tile_frag_tok(fr, 16 * q, 16 * p, l16, g), a4);
                a_[0] = a4[0]; a_[1] = a4[1]; a_[2] = a4[2]; a_[3] = a4[3];
                unpack4(tile_frag_tok(fr, 16 * q, 16 * p + 4, l16, g), nx);   // rows tk+4..: only the first is used
                a_[4] = (g == 3) ? gq : nx[0];                                  // a_16 = g
                unpack4_in<Tin>(tile_frag_tok(wt, 16 * q, 16 * p, l16, g), w_);   // (the raw tile: the input type)
                unpack4(rtq, rt_); unpack4(ktq, kt_);
            }
            const float4 vg4 = *reinterpret_cast<const float4 *>(&vgyw[4 * g]);
            const float vg_[4] = {vg4.x, vg4.y, vg4.z, vg4.w};
            float ia[5];
#pragma unroll
            for (int rr = 0; rr < 5; ++rr) ia[rr] = __builtin_amdgcn_rcpf(a_[rr]);
            float P[4], D[4], gro[4], gko[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                P[rr] = rt_[rr] * X[rr];
                D[rr] = kt_[rr] * W[rr] - P[rr];
                const float uvg = uj * vg_[rr];
                const float rraw = rt_[rr] * ia[rr], kraw = kt_[rr] * a_[rr + 1];
                gro[rr] = fmaf(a_[rr], X[rr], uvg * kraw);
                gko[rr] = fmaf(ia[rr + 1], W[rr], uvg * rraw);
                gu_acc = fmaf(rraw * kraw, vg_[rr], gu_acc);
            }
            // exclusive prefix of D over the 16 tokens: 4 in this lane, the rest in the lane groups below
            float pre = E + prefix_rows(D[0] + D[1] + D[2] + D[3], g);
            float gwo[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                // exp(w) <= kWildLimit here (anything larger sends this (b, h) to the exact second pass)
                const float ew = fast_exp(w_[rr]);
                gwo[rr] = -ew * (pre - P[rr]);
                pre += D[rr];
            }
            // the gradient of the first and the last decay is zero by definition (the flow balance
            // leaves rounding residue there); only the two tiles holding them pay for the test
            // (with a non-zero initial state / a gradient arriving at the final state they are not zero)
            if ((c == 0 && p == 0) || (c == nchunk - 1 && p == (((T - 1) >> 4) & 3))) {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                    if ((t0 + tk + rr == 0 && !a.s0) || (t0 + tk + rr == T - 1 && !a.gsT)) gwo[rr] = 0.f;
            }
            store_tile(t0 + tk, gro, gko, gwo);
            __builtin_amdgcn_sched_barrier(0);
        }
        ++item;
    };
    for (int c = nchunk - 1; c >= 0; --c) visit(c, Sraw);
    if (a.gs0 && GRP == 0) {   // the reverse state has arrived at t = 0: dL/dS_0
#pragma unroll
        for (int m = 0; m < 4; ++m)
            *reinterpret_cast<f32x4 *>(a.gs0 + (int64_t)(b * H + h) * (kN * kN) + col * kN + 16 * m + 4 * g) = Gj[m];
    }
    // gu: fold the four lane groups (different tokens, same channel), then the consumer groups
    gu_acc = sum_rows(gu_acc);
    if (GRP == 1 && g == 0) gu_lds[col] = gu_acc;
    __threadfence_block();
    __syncthreads();
    if (GRP == 0 && g == 0 && !*s_wild)     // (the exact second pass writes gu itself)
        store1(reinterpret_cast<Tout *>(a.gu) + (int64_t)b * C + h * kN + col, gu_acc + gu_lds[col]);
}

// ------------------------------------------------------------------------------------------
// gv role: wave q owns value columns i = 16q..16q+15 of the reverse state Gi (rows j).
// ------------------------------------------------------------------------------------------
struct GvState {
    f32x4 Gi[4];
    // gsT: this pair's [key][value] block or null; the copy here has rows j = 16m + 4g + rr, column i = col
    __device__ __forceinline__ void init(const float *gsT, int col, int g) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) Gi[m][rr] = gsT ? gsT[(16 * m + 4 * g + rr) * kN + col] : 0.f;
    }
};
// the tiles of chunk c (chunk visit `item`), last to first
template <typename Tout, bool kRagged>
__device__ __forceinline__ void bwd_gv_chunk(GvState &st, const BwdArgs &a, const unsigned char *smem, Tout *gv_h,
                                             uint32_t rowelems, int c, int item, int q, int lane)
{
    const int T = a.T;
    const int g = lane >> 4, l16 = lane & 15;
    f32x4 (&Gi)[4] = st.Gi;
    const unsigned char *op = smem + BwdLds::kOp + (item & 1) * BwdLds::kOpBytes;
    const unsigned char *rt = smem + BwdLds::kRawRK + (item % 3) * 2 * kTileBytes, *kt = rt + kTileBytes;
    const float *gg_ = reinterpret_cast<const float *>(op + BwdLds::kOpG);
    const float *ruk = reinterpret_cast<const float *>(op + BwdLds::kOpRuk);
    const unsigned char *gyt = smem + BwdLds::kRawVG + (item % 3) * 2 * kTileBytes + kTileBytes;
    const int t0 = c * CL;
#pragma unroll 1
    for (int pp = 3; pp >= 0; --pp) {
        const int row = 16 * pp + l16;
        const bf16x8 rf0 = tile_frag_ch(rt, row, 0, g), rf1 = tile_frag_ch(rt, row, 1, g);
        const bf16x8 kf0 = tile_frag_ch(kt, row, 0, g), kf1 = tile_frag_ch(kt, row, 1, g);
        const s16x4 gyq = tile_frag_tok(gyt, 16 * q, 16 * pp, l16, g);
        const float rukv = ruk[row];
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
            const float4 gg = *reinterpret_cast<const float4 *>(&gg_[pp * kN + 16 * m + 4 * g]);
            Gi[m][0] *= gg.x; Gi[m][1] *= gg.y; Gi[m][2] *= gg.z; Gi[m][3] *= gg.w;
        }
        // the products are formed transposed (accumulator rows i = 4g + r, column s = l16): a lane holds
        // four neighbouring channels of one token and writes them with one 8-byte store
        f32x4 GV = {0.f, 0.f, 0.f, 0.f};
        GV = mfma16(gyq, pack4(A), GV);
        chain_gap(GV);
        GV = mfma32(acc_as_operand(Gi[0], Gi[1]), kf0, GV);
        GV = mfma32(acc_as_operand(Gi[2], Gi[3]), kf1, GV);
#pragma unroll
        for (int m = 0; m < 4; ++m) Gi[m] = mfma16(tile_frag_tok(rt, 16 * m, 16 * pp, l16, g), gyq, Gi[m]);
        settle(GV, Gi);
        {
            const int t = t0 + row;   // channels 16q + 4g .. +3 of this token
            if (!kRagged || t < T) store4(gv_h + ((uint32_t)t * rowelems + (uint32_t)(16 * q + 4 * g)), GV[0], GV[1], GV[2], GV[3]);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Loader / producer: wave p <-> tile p of every chunk, lane = channel.
// ------------------------------------------------------------------------------------------
template <typename Tin, bool kRagged>
__device__ __forceinline__ void bwd_producer(const BwdArgs &a, unsigned char *smem, int *s_wild, int pair0, int p, int lane)
{
    const int T = a.T, H = a.H;
    const int ch = lane;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + CL - 1) / CL;
    // item = chunk visit: from chunk n-1 down to 0
    const int h = pair0 % H, b0 = pair0 / H;
    const int nitem = nchunk;
    typedef typename OutOf<Tin>::type Tout;
    const float uc = load1(reinterpret_cast<const Tin *>(a.u) + h * kN + ch);
    const uint32_t rowbytes = (uint32_t)C * 2u;
    const uint32_t lds0 = lds_address(smem);
    // Where an item is: which chunk.  Loads, operand preparation and the gv role each walk the item
    // sequence with a cursor of their own.
    struct Cursor {
        int c;
    };
    // the rows of the pair
    const int64_t base0 = (int64_t)b0 * T * C + (int64_t)h * kN;
    const bf16_t *rb = a.r + base0, *kb_ = a.k + base0, *vb = a.v + base0, *wb = a.w + base0, *gb = a.gy + base0;   // loads
    const bf16_t *ckb = reinterpret_cast<const bf16_t *>(a.ckpt + (int64_t)(b0 * H + h) * nchunk * (kN * kN));      // state loads
    Tout *gvb = reinterpret_cast<Tout *>(a.gv) + base0;                                                            // gv role
    // this lane's part of an 8-row block load: row (lane >> 3), 16-byte piece swizzled with the row
    const int lrow = lane >> 3;
    const uint32_t lpiece = (uint32_t)(((lane & 7) ^ lrow) << 4);
    // Rows past the end of the sequence are fetched from row T-1 (valid memory); the preparation
    // turns them into r = k = 0, w = -inf (decay 1), and the v, gy rows only ever meet zero operands.
    // Returns the number of loads.
    auto issue_loads = [&](int it, const Cursor &cu) -> int {
        const int tb = cu.c * CL + 16 * p;
        const uint32_t rk = lds0 + BwdLds::kRawRK + (it % 3) * 2 * kTileBytes + 16 * p * kTileRow;
        const uint32_t ww = lds0 + BwdLds::kRawW + (it % 3) * kTileBytes + 16 * p * kTileRow;
        const uint32_t vg = lds0 + BwdLds::kRawVG + (it % 3) * 2 * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int t = tb + 8 * hf + lrow;
            const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + lpiece;
            load_rows8_to_lds(kb_, o, rk + kTileBytes + 8 * hf * kTileRow);
            load_rows8_to_lds(wb, o, ww + 8 * hf * kTileRow);
            load_rows8_to_lds(vb, o, vg + 8 * hf * kTileRow);
            load_rows8_to_lds(rb, o, rk + 8 * hf * kTileRow);
            load_rows8_to_lds(gb, o, vg + kTileBytes + 8 * hf * kTileRow);
        }
        return 10;
    };
    // The saved forward state of item `it`: the
    // chunk's 64x64 bf16 block [i][j] is a tile with i in the place of the token; wave p brings rows
    // 16p..16p+15.  It is requested ONE item ahead (two slots), ahead of the tile loads in the queue,
    // and awaited at the end of the visit, behind the gv stores issued in between -- the consumer
    // waves, which would otherwise load it behind their own gradient stores and wait for those to
    // reach the L2, then have no load to wait for at all.
    auto issue_state = [&](int it, const Cursor &cu) {
        const bf16_t *src = ckb + (int64_t)cu.c * (kN * kN);
        const uint32_t dst = lds0 + BwdLds::kState + (it & 1) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
            load_rows8_to_lds(src, (uint32_t)((16 * p + 8 * hf + lrow) * kTileRow) + lpiece, dst + 8 * hf * kTileRow);
    };
    // Waits for this wave's tile loads of one item.  `n` = operations issued after them: the loads
    // of the following item and, with the gv role on this wave, the 4 gv stores of the chunk
    // visit in between (memory operations of a wave complete in program order; the stores are left
    // in flight -- waiting for them costs more than a microsecond per chunk under load).
    auto wait_younger = [&](int n) {
        switch (n) {   // tile loads {0, 10} + state loads {0, 2} + gv stores {0, 4}
        case 16: wait_loads<16>(); break;
        case 14: wait_loads<14>(); break;
        case 12: wait_loads<12>(); break;
        case 10: wait_loads<10>(); break;
        case 6: wait_loads<6>(); break;
        case 4: wait_loads<4>(); break;
        case 2: wait_loads<2>(); break;
        default: wait_loads<0>(); break;
        }
    };
    // per-lane byte offsets of channel `ch` inside a tile row, for the 8 swizzle phases
    uint32_t choff[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) choff[s] = (uint32_t)((((ch >> 3) ^ s) << 4) + ((ch & 7) << 1)) + (uint32_t)(16 * p * kTileRow);
    const float kLog2Log2e = 0.5287663729448977f;   // log2(log2(e)): exp(w) log2(e) = 2^(w log2(e) + this)
    auto prepare = [&](int it, const Cursor &cu) {
        const int tb = cu.c * CL + 16 * p;
        // lane addresses of the 8 swizzle phases in the three blocks this item uses (the row and tensor
        // offsets on top of them are instruction immediates)
        unsigned char *a_rk[8];
        const unsigned char *a_w[8];
        unsigned char *a_op[8];
#pragma unroll
        for (int sw = 0; sw < 8; ++sw) {
            a_rk[sw] = smem + (BwdLds::kRawRK + (it % 3) * 2 * kTileBytes + choff[sw]);
            a_w[sw] = smem + (BwdLds::kRawW + (it % 3) * kTileBytes + choff[sw]);
            a_op[sw] = smem + (BwdLds::kOp + (it & 1) * BwdLds::kOpBytes + choff[sw]);
        }
        float fr[16], fk[16], fw[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            uint32_t ra = *reinterpret_cast<const uint16_t *>(a_rk[e & 7] + e * kTileRow);
            uint32_t rk = *reinterpret_cast<const uint16_t *>(a_rk[e & 7] + kTileBytes + e * kTileRow);
            uint32_t rw = *reinterpret_cast<const uint16_t *>(a_w[e & 7] + e * kTileRow);
            if (kRagged && tb + e >= T) { ra = 0u; rk = 0u; rw = neg_inf_bits<Tin>(); }
            fr[e] = in_bits_to_float<Tin>(ra); fk[e] = in_bits_to_float<Tin>(rk); fw[e] = in_bits_to_float<Tin>(rw);
        }
        // exponents are kept in base 2 (one v_exp_f32 each, no extra scaling multiply)
        float xr[16], xk[16], pr[16], fa[16];
        float cs2 = 0.f, pa = 1.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float ew2 = exp2_fast(fmaf(fw[e], kLog2e, kLog2Log2e));   // exp(w) * log2(e)
            fa[e] = pa;
            xr[e] = fr[e] * pa;
            cs2 += ew2;
            xk[e] = fk[e] * exp2_fast(cs2);
            pa *= exp2_fast(-ew2);
            pr[e] = fr[e] * uc * fk[e];
        }
        if (__builtin_amdgcn_ballot_w64(!(cs2 <= kWildLimit * kLog2e)) != 0ull) {
            if (lane == 0) *s_wild = 1;
        }
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const uint32_t pr2 = pack_bf16x2(xr[e], xr[e + 1]), pk2 = pack_bf16x2(xk[e], xk[e + 1]);
            const uint32_t pf2 = pack_bf16x2(fa[e], fa[e + 1]);
            unsigned char *o0 = a_op[e & 7] + e * kTileRow, *o1 = a_op[(e + 1) & 7] + (e + 1) * kTileRow;
            unsigned char *q0 = a_rk[e & 7] + e * kTileRow, *q1 = a_rk[(e + 1) & 7] + (e + 1) * kTileRow;
            // R~ and K~ take the place of the raw r and k this lane read above
            *reinterpret_cast<uint16_t *>(q0) = (uint16_t)pr2;
            *reinterpret_cast<uint16_t *>(q1) = (uint16_t)(pr2 >> 16);
            *reinterpret_cast<uint16_t *>(q0 + kTileBytes) = (uint16_t)pk2;
            *reinterpret_cast<uint16_t *>(q1 + kTileBytes) = (uint16_t)(pk2 >> 16);
            *reinterpret_cast<uint16_t *>(o0 + BwdLds::kOpFr) = (uint16_t)pf2;
            *reinterpret_cast<uint16_t *>(o1 + BwdLds::kOpFr) = (uint16_t)(pf2 >> 16);
        }
        unsigned char *op = smem + BwdLds::kOp + (it & 1) * BwdLds::kOpBytes;
        reinterpret_cast<float *>(op + BwdLds::kOpG)[p * kN + ch] = pa;
        const float tr = transpose_reduce16(pr, lane);
        if ((lane & 3) == 0) reinterpret_cast<float *>(op + BwdLds::kOpRuk)[16 * p + ((lane >> 2) & 15)] = tr;
    };
    // item `it` is loaded during iteration it-2 (or the prologue) and prepared during iteration it-1
    GvState gvst;
    gvst.init(a.gsT ? a.gsT + (int64_t)(b0 * H + h) * (kN * kN) : nullptr, 16 * p + (lane & 15), lane >> 4);
    // every item's saved state is loaded one item ahead
    auto state_by_load = [&](int it) { return it < nitem; };
    // gv stores an item's visit leaves in flight behind the loads issued before them.  The chunk with
    // the ragged tail issues anything from 0 to 4 (a store whose lanes are all past the end is
    // skipped): counting none for it makes the waits behind it wait for everything older.
    auto gv_stores = [&](const Cursor &cu) { return (kRagged && cu.c == nchunk - 1) ? 0 : 4; };
    Cursor cur_l = {nchunk - 1}, cur_p = cur_l, cur_v = cur_l;   // items it+2 (loads), it+1 (state, preparation), it (gv)
    auto next_load_item = [&]() { --cur_l.c; };
    auto next_prepared_item = [&]() { --cur_p.c; };
    if (state_by_load(0)) issue_state(0, cur_p);
    issue_loads(0, cur_l);
    next_load_item();
    int first_younger = 0;
    if (nitem > 1) { first_younger = issue_loads(1, cur_l); next_load_item(); }
    wait_younger(first_younger);
    prepare(0, cur_p);
    next_prepared_item();
    int gv_stores_before = 0;   // gv stores of item it-1
    for (int it = 0; it < nitem; ++it) {
        __syncthreads();
        // free again: the r, k block of item it-1 and the raw w, v, gy blocks of item it-1 (read by the
        // other roles before the barrier), and the state tile of item it-1
        const int state_loads = state_by_load(it + 1) ? 2 : 0;
        if (state_loads) issue_state(it + 1, cur_p);
        int younger = 0;
        if (it + 2 < nitem) { younger = issue_loads(it + 2, cur_l); next_load_item(); }
        if (it + 1 < nitem) {
            wait_younger(younger + state_loads + gv_stores_before);
            prepare(it + 1, cur_p);
            next_prepared_item();
        }
        // the gv role, on the waves the operand preparation leaves partly idle
        bwd_gv_chunk<Tout, kRagged>(gvst, a, smem, gvb, (uint32_t)C, cur_v.c, it, p, lane);
        gv_stores_before = gv_stores(cur_v);
        // the next item's state has to be in LDS when the consumers pass the barrier
        if (state_loads) wait_younger(younger + gv_stores_before);
        --cur_v.c;
    }
    wait_loads<0>();
    __threadfence_block();
    __syncthreads();
}

// Wave layout: 12 waves, four per role, one wave of each role per SIMD:
//   loader/producer + gv | consumer group 0 (tiles 3, 1) | consumer group 1 (tiles 2, 0)
constexpr int kBwdWaves = 12;

template <typename Tin, bool kRagged>
__global__ __launch_bounds__(kBwdWaves * 64) void chunk_bwd_kernel(BwdArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild[1];    // a tile of this workgroup's pair left the chunked form's range
    __shared__ float s_ft[kN];   // exact second pass with state gradients: the anchor of the gw sums
    static_assert(sizeof(ScanBwdALds) <= BwdLds::kBytes && sizeof(ScanBwdBLds) <= BwdLds::kBytes,
                  "the exact second pass reuses the LDS block");
    if (threadIdx.x == 0) s_wild[0] = 0;
    __syncthreads();

    const int pair0 = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int role = wave >> 2, q = wave & 3;
    typedef typename OutOf<Tin>::type Tout;
    if (role == 0) bwd_producer<Tin, kRagged>(a, smem, s_wild, pair0, q, lane);
    else if (role == 1) bwd_consumer<Tin, kRagged, 0>(a, smem, s_wild, pair0, q, lane);
    else bwd_consumer<Tin, kRagged, 1>(a, smem, s_wild, pair0, q, lane);
    // exact second pass for a (b, h) if any of its tiles left the representable range; the
    // pair's own slice of the state workspace (nchunk x 64 x 64 floats = T' x 64) holds P
    if (s_wild[0]) {
        const int b = pair0 / a.H, h = pair0 % a.H;
        const int nchunk = (a.T + CL - 1) / CL;
        float *ck = a.ckpt + (int64_t)(b * a.H + h) * nchunk * (kN * kN);
        const int64_t so = (int64_t)(b * a.H + h) * (kN * kN);
        const float *s0p = a.s0 ? a.s0 + so : nullptr, *gsTp = a.gsT ? a.gsT + so : nullptr;
        const bool states = a.s0 || a.gsT || a.gs0;
        __syncthreads();
        auto in = [](const void *p) { return reinterpret_cast<const Tin *>(p); };
        auto out = [](void *p) { return reinterpret_cast<Tout *>(p); };
        const Tout *gyp = reinterpret_cast<const Tout *>(a.gy_orig);
        scan_bwd_a_body<Tin, Tout>(*reinterpret_cast<ScanBwdALds *>(smem), b, h, a.T, a.H, in(a.r), in(a.k), in(a.v_orig), in(a.w), in(a.u), gyp,
                                   out(a.gr), out(a.gu), ck, kN, s0p, gsTp, states ? s_ft : nullptr);
        __threadfence_block();
        __syncthreads();
        scan_bwd_b_body<Tin, Tout>(*reinterpret_cast<ScanBwdBLds *>(smem), b, h, a.T, a.H, in(a.r), in(a.k), in(a.v_orig), in(a.w), in(a.u), gyp, ck, kN,
                                   out(a.gk), out(a.gv), out(a.gw), gsTp, states ? s_ft : nullptr, a.gs0 ? a.gs0 + so : nullptr, a.s0 == nullptr);
        __syncthreads();
    }
    // Fused batch sum of gu (what the caller otherwise does with one more kernel): the workgroup that
    // is the last of its head to deliver adds up the B partials.  The partials travel as written-
    // through (agent scope) stores into the unused second half of each workgroup's workspace slice,
    // completed before the arrival counter is bumped; no fence, which would write back the whole L2.
    if (a.gu_sum != nullptr) {
        __shared__ int s_last;
        const int h = pair0 % a.H;
        const int nchunk = (a.T + CL - 1) / CL;
        const int64_t slice = (int64_t)nchunk * (kN * kN), C = (int64_t)a.H * kN;
        const int nparts = a.B;   // what adds up to the head's sum: one partial per batch row
        __threadfence_block();   // this workgroup's gu rows (consumer group 0 or the second pass) are written
        __syncthreads();
        const int tid = threadIdx.x;
        if (tid < kN) {          // wave 0
            const float part = load1(reinterpret_cast<const Tout *>(a.gu) + (int64_t)(pair0 / a.H) * C + h * kN + tid);
            __hip_atomic_store(a.ckpt + (int64_t)pair0 * slice + slice / 2 + tid, part, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (tid == 0)
                s_last = __hip_atomic_fetch_add(a.arrivals + h, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nparts - 1;
        }
        __syncthreads();
        if (s_last && tid < kN) {
            float acc = 0.f;
            for (int j = 0; j < nparts; ++j)
                acc += __hip_atomic_load(a.ckpt + (int64_t)(h + j * a.H) * slice + slice / 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            store1(reinterpret_cast<Tout *>(a.gu_sum) + h * kN + tid, acc);
            if (tid == 0) __hip_atomic_store(a.arrivals + h, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // armed again
        }
    }
}

size_t chunk_backward_workspace_bytes(int64_t B, int64_t T, int64_t H) {
    const int64_t nchunk = (T + CL - 1) / CL;
    return (size_t)(B * H * nchunk) * kN * kN * sizeof(float);
}
size_t chunk_saved_bytes(int64_t B, int64_t T, int64_t H) {
    return chunk_backward_workspace_bytes(B, T, H) + (((size_t)H * sizeof(int) + 255) & ~(size_t)255);
}

template <typename T>
__global__ void sum_over_batch_kernel(int B, int C, const T *__restrict__ p, T *__restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float acc = 0.f;
    for (int b = 0; b < B; ++b) acc += load1(p + (int64_t)b * C + c);
    store1(out + c, acc);
}
hipError_t sum_over_batch(hipStream_t st, int out_dtype, int64_t B, int64_t C, const void *partials, void *sum) {
    const dim3 grid((unsigned)((C + 255) / 256)), block(256);
    if (out_dtype == kBF16)
        hipLaunchKernelGGL(sum_over_batch_kernel<bf16_t>, grid, block, 0, st, (int)B, (int)C, (const bf16_t *)partials, (bf16_t *)sum);
    else
        hipLaunchKernelGGL(sum_over_batch_kernel<float>, grid, block, 0, st, (int)B, (int)C, (const float *)partials, (float *)sum);
    return hipGetLastError();
}

hipError_t chunk_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, bool states_ready,
                          void *gu_sum, const float *s0, const float *gsT, float *gs0,
                          int in_dtype, const void *v_orig, const void *gy_orig)
{
    const size_t lds = BwdLds::kBytes;
    BwdArgs a;
    a.v_orig = v_orig ? v_orig : v; a.gy_orig = gy_orig ? gy_orig : gy;
    a.s0 = s0; a.gsT = gsT; a.gs0 = gs0;
    a.T = (int)T; a.H = (int)H;
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w;
    a.u = (const bf16_t *)u; a.gy = (const bf16_t *)gy;
    a.gr = (bf16_t *)gr; a.gk = (bf16_t *)gk; a.gv = (bf16_t *)gv; a.gw = (bf16_t *)gw; a.gu = (bf16_t *)gu;
    a.ckpt = (float *)workspace;
    a.B = (int)B;
    a.gu_sum = states_ready ? (bf16_t *)gu_sum : nullptr;
    a.arrivals = reinterpret_cast<int *>(reinterpret_cast<char *>(workspace) + chunk_backward_workspace_bytes(B, T, H));
    const unsigned grid = (unsigned)(B * H);
    auto launch_in = [&](auto in_tag, auto ragged_tag) -> hipError_t {
        constexpr auto kern = chunk_bwd_kernel<decltype(in_tag), decltype(ragged_tag)::value>;
        hipError_t e = allow_dynamic_lds<kern>((int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kBwdWaves * 64), lds, st, a);
        return hipGetLastError();
    };
    auto launch = [&](auto ragged_tag) -> hipError_t {
        // fp16 tensors (fp32 gradients): only with saved states, v and gy as bf16 copies plus the originals
        if (in_dtype == kF16) return states_ready && v_orig && gy_orig ? launch_in(f16_t{}, ragged_tag) : hipErrorInvalidValue;
        return launch_in(bf16_t{}, ragged_tag);
    };
    const bool ragged = (T % CL) != 0;   // the last chunk has tokens past the end
    // (gradients through the state: the block form takes them with one pair per workgroup)
    const bool block_form = in_dtype == kBF16 && block_backward_applies(B, T, H) && ((!s0 && !gsT && !gs0) || B * H <= block_grid(B, H));
    if (!states_ready) {
        // No states from a saving forward: the forward kernel's state-only pass (no y) leaves them in
        // the workspace first.
        hipError_t e = chunk_forward(st, kF32, B, T, H, r, k, v, w, u, s0, nullptr, nullptr, nullptr, workspace, nullptr, false, false);
        if (e != hipSuccess) return e;
    }
    if (block_form) return block_backward(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace, a.gu_sum, s0, gsT, gs0);
    return ragged ? launch(std::true_type{}) : launch(std::false_type{});
}

// Training pair in time segments, last step: gu of a batch row = sum over its segments; the decay
// gradient at the first and the last token of a sequence is zero by definition
// (rwkv_kernels.cu:381,406), where the kernels, given explicit states, leave rounding residue.
__global__ void segments_finish_kernel(int P, int64_t T, int C, const bf16_t *__restrict__ gu_rows,
                                       bf16_t *__restrict__ gu, bf16_t *__restrict__ gw, bool zero_first, bool zero_last)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= C) return;
    float acc = 0.f;
    for (int p = 0; p < P; ++p) acc += load1(gu_rows + ((int64_t)b * P + p) * C + c);
    store1(gu + (int64_t)b * C + c, acc);
    if (zero_first) store1(gw + (int64_t)b * T * C + c, 0.f);
    if (zero_last) store1(gw + ((int64_t)b * T + T - 1) * C + c, 0.f);
}

hipError_t chunk_backward_saved_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                                         void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum,
                                         void *saved, void *extra)
{
    const TrainSegments s = train_segments_layout(B, T, H, extra);
    const int64_t L = T / s.P, rows = B * s.P;
    // (1) What each segment alone sends back into its incoming state: G_0 = sum_t (prod_{s<t} d_s) r_t^T gy_t.
    // That is the state the FORWARD recurrence builds from zero over the segment read back to front
    // with r in the place of k and gy in the place of v, so the forward kernel's state-only pass does it.
    hipError_t e = chunk_forward(st, kF32, rows, L, H, r, r, gy, w, u, nullptr, nullptr, nullptr, s.gstates, nullptr, nullptr, true);
    if (e != hipSuccess) return e;
    // (2) chained backwards in time: the gradient arriving at the end of every segment
    if ((e = segment_chain_reverse(st, s.P, B, H, s.dsum, s.gstates)) != hipSuccess) return e;
    // (3) every segment again, between its true incoming state and its true arriving gradient
    e = chunk_backward(st, rows, L, H, r, k, v, w, u, gy, gr, gk, gv, gw, s.gu_rows, saved, true, gu_sum,
                       s.states, s.gstates, nullptr);
    if (e != hipSuccess) return e;
    const int C = (int)(H * kN);
    hipLaunchKernelGGL(segments_finish_kernel, dim3((unsigned)((C + 255) / 256), (unsigned)B), dim3(256), 0, st,
                       s.P, T, C, (const bf16_t *)s.gu_rows, (bf16_t *)gu, (bf16_t *)gw, true, true);
    return hipGetLastError();
}

// The same with an initial state, a gradient arriving at the final state and dL/dS_0 wanted
// (wkv6_backward_with_state): nothing was saved by a forward pass, so the segments' incoming
// states and the chunk states are rebuilt first (state-only passes of the forward kernel).
hipError_t chunk_backward_state_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                         const void *r, const void *k, const void *v, const void *w, const void *u,
                                         const float *s0, const void *gy, const float *gsT,
                                         void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0,
                                         void *saved, void *extra)
{
    const TrainSegments s = train_segments_layout(B, T, H, extra);
    const int64_t L = T / s.P, rows = B * s.P;
    hipError_t e = chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, nullptr, nullptr, nullptr, s.states, nullptr, s.dsum);
    if (e != hipSuccess) return e;
    if ((e = segment_chain_forward(st, s.P, B, H, s.dsum, s.states, s0)) != hipSuccess) return e;
    e = chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, s.states, nullptr, nullptr, nullptr, saved, nullptr, false, false);
    if (e != hipSuccess) return e;
    e = chunk_forward(st, kF32, rows, L, H, r, r, gy, w, u, nullptr, nullptr, nullptr, s.gstates, nullptr, nullptr, true);
    if (e != hipSuccess) return e;
    if ((e = segment_chain_reverse(st, s.P, B, H, s.dsum, s.gstates, gsT, gs0)) != hipSuccess) return e;
    e = chunk_backward(st, rows, L, H, r, k, v, w, u, gy, gr, gk, gv, gw, s.gu_rows, saved, true, nullptr,
                       s.states, s.gstates, nullptr);
    if (e != hipSuccess) return e;
    const int C = (int)(H * kN);
    // (the decay gradient at an end of the sequence is zero by definition only where no state / no gradient comes in)
    hipLaunchKernelGGL(segments_finish_kernel, dim3((unsigned)((C + 255) / 256), (unsigned)B), dim3(256), 0, st,
                       s.P, T, C, (const bf16_t *)s.gu_rows, (bf16_t *)gu, (bf16_t *)gw, s0 == nullptr, gsT == nullptr);
    return hipGetLastError();
}

}  // namespace wkv6
