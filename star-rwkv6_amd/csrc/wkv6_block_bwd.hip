// WKV6 backward in block form for gfx950 (bf16 MFMA, fp32 states).  Same cases as the block-form
// forward (wkv6_block_fwd.hip: bf16 tensors, more than half a (batch, head) pair per compute unit;
// kMulti: several pairs per workgroup, one after the other through one pipeline; kRagged: a sequence
// length that is no multiple of 64), without gradients through the state; the tile form in
// wkv6_chunk_bwd.hip serves every other case.  The forward state at every chunk start comes from the
// workspace (bf16, transposed: [chunk][i][j]).  Notation and the operand scaling are in wkv6_block.h.
//
// Per block of 32 tokens (t, s local; G = reverse state arriving at the block's END from the future,
// rows j; S = forward state at the block's start; alpha, g1, g2 of the block):
//   dA[t][s] = gy_t . v_s (s < t)                A[t][s] = R~_t . K~_s (s < t),  A[t][t] = sum_j r u k
//   X[t][j]  = sum_s dA[t][s] K~_s[j] + g1_j sum_i gy_t[i] S[j][i]           gr'_t = alpha_t X_t
//   W[s][j]  = sum_t dA[t][s] R~_t[j] + g2_j sum_i v_s[i] G[j][i]            gk'_s = W_s / alpha_{s+1}
//   gv_s[i]  = sum_t A[t][s] gy_t[i] + sum_j K~_s[j] g2_j G[j][i]
//   G       <- g1 o (g2 o G + R~^T gY)
//   gr = gr' + u k <v,gy>,  gk = gk' + u r <v,gy>,  gu[j] = sum_t r k <v,gy>
//   gw_t[j]  = -exp(w_t[j]) ( E[j] + sum_{m<t} (Q_m - P_m) - P_t ),   P = R~ X,  Q = K~ W,
//   E[j] = sum_i S[j][i] G_new[j][i]       (the flow balance across decay step t, anchored at the block start)
// Both states are touched twice per block; everything between is dense 16x16 block work on the
// matrix cores plus one elementwise pass over the (token, channel) grid.
//
// Workgroup: 12 waves.
//   Four producer waves (wave p <-> tokens 16p..16p+15): bring the raw r, k, w, v, gy rows of a chunk
//       straight into LDS two visits ahead and the chunk's saved state one visit ahead; one visit
//       ahead turn r, k, w into R~, K~ (over the raw r, k), exp(w) (over the raw w), alpha, g1, g2 and
//       the diagonal; then run the gv role (wave q <-> value columns 16q..), which takes g2 o G of each
//       block from LDS, where the other waves publish it as ready MFMA operands.
//   Eight waves (q, half) <-> key channels 16q..16q+15, block `half` of the visit: X, W and the
//       elementwise pass (gr, gk, gw, gu), products formed transposed (a lane holds four neighbouring
//       channels of one token; two 16-token row groups are paired through a lane-row swap so that every
//       gradient leaves as 16-byte stores).  Each carries a copy of G with rows i through both blocks; the
//       wave of the later block also steps the saved state over the earlier block to get its S.
#include "wkv6_mfma.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"
#include "wkv6_block.h"

#include <type_traits>

namespace wkv6 {

struct BlockBwdLds {
    static constexpr int kRawRK = 0;                                   // [item % 3][r, k] raw tiles, turned into R~, K~ in place
    static constexpr int kRawW = kRawRK + 3 * 2 * kTileBytes;          // [item % 3] raw w tiles, turned into exp(w) in place
    static constexpr int kRawVG = kRawW + 3 * kTileBytes;              // [item & 1][v, gy] raw tiles
    static constexpr int kAlpha = kRawVG + 2 * 2 * kTileBytes;         // [item & 1] row t: alpha_{t+1}
    static constexpr int kVec = kAlpha + 2 * kTileBytes;               // [item & 1] per-visit vectors
    static constexpr int kState = kVec + 2 * kBlockVecBytes;           // [item & 1] saved forward state of the chunk, bf16 [i][j] as a tile
    static constexpr int kScratch = kState + 2 * kTileBytes;           // [8 waves][16] floats
    static constexpr int kGu = kScratch + 8 * 16 * 4;                  // [2 pair parities][2 halves][64] floats: gu partials of a pair; [64]: gu summed over the workgroup's pairs
    static constexpr int kGFlags = kGu + 5 * kN * 4;                       // [2 blocks][4 q] visit number + 1 once the wave has written its columns of kGt
    static constexpr int kGt = kGFlags + 64;                           // [2 blocks] g2 o G at the block's end, bf16 [j][i] tiles (what gv and W take)
    static constexpr int kBytes = kGt + 2 * kTileBytes;
};
static_assert(BlockBwdLds::kBytes <= 160 * 1024, "LDS block of the block-form backward kernel");

struct BlockBwdArgs {
    int T, H, B;
    int bstep;        // batch rows between two pairs of a workgroup (B: one pair per workgroup)
    const bf16_t *r, *k, *v, *w, *u, *gy;
    bf16_t *gr, *gk, *gv, *gw, *gu;
    bf16_t *gu_sum;   // null, or C elements: receives the sum of gu over the batch
    int *arrivals;    // per head: workgroups that have delivered their gu partial (zero on entry)
    float *ckpt;
    // gradients through the state (all null for the stateless operator, and with several pairs per workgroup):
    // fp32 (B,H,64,64) [key][value]
    const float *s0, *gsT;   // initial state (the saved chunk states start from it); gradient arriving at the final state
    float *gs0;              // receives dL/dS_0
};

// inclusive prefix over the 16 lanes of a row (tokens), per lane value
__device__ __forceinline__ float scan_row16(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xF, 0xF, true));   // row_shr:1
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x112, 0xF, 0xF, true));   // row_shr:2
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x114, 0xF, 0xF, true));   // row_shr:4
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x118, 0xF, 0xF, true));   // row_shr:8
    return x;
}
// the value of lane 15 of the row, in every lane of the row
__device__ __forceinline__ float last_of_row16(float x) {
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(x), 0x10 | (0x0F << 5)));
}
// the value of the previous lane of the row (lane 0 of a row receives `first`)
__device__ __forceinline__ float prev_in_row16(float x, float first) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(first), __float_as_int(x), 0x111, 0xF, 0xF, false));
}

typedef volatile int __attribute__((address_space(3))) *LdsFlag;

// ------------------------------------------------------------------------------------------
// Wave (q, HALF): key channels j = 16q .. 16q+15, block HALF of the visit (tokens 32 HALF .. +31):
// gr, gk, gw, gu.  Gj[m]: reverse state, rows i = block_row_channel(m, g) + rr, column j = 16q + l16.
// ------------------------------------------------------------------------------------------
template <int HALF, bool kMulti, bool kRagged>
__device__ __forceinline__ void block_bwd_xw(const BlockBwdArgs &a, unsigned char *smem, const int *s_wild, int pair0, int q, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int col = 16 * q + l16;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + kBlockTokens - 1) / kBlockTokens;
    const int b0 = pair0 / H, h = pair0 - b0 * H;
    const int npw = kMulti ? (a.B - b0 + a.bstep - 1) / a.bstep : 1;   // pairs of this workgroup: batch rows b0, b0 + bstep, ... (one head)
    const int nvisit = npw * nchunk;
    const uint32_t rowbytes = (uint32_t)C * 2u;
    const int64_t base0 = (int64_t)b0 * T * C + (int64_t)h * kN;
    char *gr_h = reinterpret_cast<char *>(a.gr + base0), *gk_h = reinterpret_cast<char *>(a.gk + base0), *gw_h = reinterpret_cast<char *>(a.gw + base0);
    f32x4 Gj[4];
    // the reverse state a pair starts from: zero, or the gradient arriving at its final state ([key j][value i])
    const float *const gsT = kMulti ? nullptr : a.gsT;   // (state gradients: one pair per workgroup only)
    float *const gs0 = kMulti ? nullptr : a.gs0;
    const bool has_s0 = !kMulti && a.s0 != nullptr;
    auto start_G = [&](int slot_) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            Gj[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
            if (gsT) Gj[m] = *reinterpret_cast<const f32x4 *>(gsT + (int64_t)((b0 + slot_ * a.bstep) * H + h) * (kN * kN) + col * kN + block_row_channel(m, g));
        }
    };
    start_G(0);
    float u4[4];
    load4(a.u + h * kN + 16 * q + 4 * g, u4);   // u of this lane's four channels 16q + 4g + rr
    float gu_acc[4] = {0.f, 0.f, 0.f, 0.f};
    float pend = 1.f;   // per-column factor the reverse state Gj has still to be multiplied with
    // gu of a pair: both halves leave their part in LDS (rows of the pair's parity); after the next barrier
    // half 0 adds them, stores the pair's row and adds it, as stored, to the sum over the workgroup's pairs
    // (for the fused batch sum; a lane owns its four channels of that row)
    float *gu_lds = reinterpret_cast<float *>(smem + BlockBwdLds::kGu);
    auto deliver_gu = [&](int done) {   // done: number of the pair
        if (l16 == 0 && !s_wild[done]) {   // (the exact second pass writes a pair's gu itself)
            const float *rows = gu_lds + (done & 1) * 2 * kN + 16 * q + 4 * g;
            const float4 x = *reinterpret_cast<const float4 *>(rows), y = *reinterpret_cast<const float4 *>(rows + kN);
            const float t0 = x.x + y.x, t1 = x.y + y.y, t2 = x.z + y.z, t3 = x.w + y.w;
            store4(a.gu + (int64_t)(b0 + done * a.bstep) * C + h * kN + 16 * q + 4 * g, t0, t1, t2, t3);
            const uint32_t p01 = pack_bf16x2(t0, t1), p23 = pack_bf16x2(t2, t3);
            float4 *sum = reinterpret_cast<float4 *>(gu_lds + 4 * kN + 16 * q + 4 * g);
            float4 acc = *sum;
            acc.x += __uint_as_float(p01 << 16); acc.y += __uint_as_float(p01 & 0xffff0000u);
            acc.z += __uint_as_float(p23 << 16); acc.w += __uint_as_float(p23 & 0xffff0000u);
            *sum = acc;
        }
    };
    if (HALF == 0 && l16 == 0) *reinterpret_cast<float4 *>(gu_lds + 4 * kN + 16 * q + 4 * g) = make_float4(0.f, 0.f, 0.f, 0.f);
    float *scratch = reinterpret_cast<float *>(smem + BlockBwdLds::kScratch) + (4 * HALF + q) * 16;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const BlockLane la(l16, g);
    const uint32_t la_state = block_lane_state(q, l16, g), la_cols = block_lane_cols4(q, l16, g);
    const uint32_t gt_lo = tile_off(col, 8 * g), gt_hi = tile_off(col, 32 + 8 * g);
    LdsFlag g_flags = (LdsFlag)(smem + BlockBwdLds::kGFlags);
    int cv = 0, slot = 0;   // visit `it` is the cv-th visit of pair number `slot`: chunk nchunk-1-cv
    for (int it = 0; it < nvisit; ++it) {
        const int c = nchunk - 1 - cv;
        __syncthreads();
        if (kMulti && HALF == 0 && cv == 0 && slot > 0) deliver_gu(slot - 1);
        if (kMulti && cv == 0 && slot > 0) {   // a new pair: its rows, the reverse state from zero
            const int64_t base = (int64_t)(b0 + slot * a.bstep) * T * C + (int64_t)h * kN;
            gr_h = reinterpret_cast<char *>(a.gr + base); gk_h = reinterpret_cast<char *>(a.gk + base); gw_h = reinterpret_cast<char *>(a.gw + base);
            start_G(slot);
            pend = 1.f;
            gu_acc[0] = gu_acc[1] = gu_acc[2] = gu_acc[3] = 0.f;
        }
        const unsigned char *rt = smem + BlockBwdLds::kRawRK + (it % 3) * 2 * kTileBytes, *kt = rt + kTileBytes;
        const unsigned char *wt = smem + BlockBwdLds::kRawW + (it % 3) * kTileBytes;
        const unsigned char *vt = smem + BlockBwdLds::kRawVG + (it & 1) * 2 * kTileBytes, *gyt = vt + kTileBytes;
        const unsigned char *at = smem + BlockBwdLds::kAlpha + (it & 1) * kTileBytes;
        const float *vec = reinterpret_cast<const float *>(smem + BlockBwdLds::kVec + (it & 1) * kBlockVecBytes);
        const unsigned char *stt = smem + BlockBwdLds::kState + (it & 1) * kTileBytes;
        // per-column (this lane's j) factors of both blocks, and the per-row ones of this wave's block
        const float g1c0 = vec[col], g2c0 = vec[kN + col], g1c1 = vec[2 * kN + col], g2c1 = vec[3 * kN + col];
        const float4 g1r = *reinterpret_cast<const float4 *>(&vec[2 * HALF * kN + 16 * q + 4 * g]);
        // the chunk's saved state: S0[j = col][i = block_row_channel(m, g) + e]
        u32x2 Sraw[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) Sraw[m] = block_state_frag_at(stt, la_state, m);
        // One step of the reverse state over block `blk`; leaves g2 o G (what W of that block takes) as operands.
        bf16x8 GmL, GmH;
        auto step_G = [&](int blk, float g1c, float g2c, bool keep_operand) {
            const float f = pend * g2c;   // (the g1 of the step before is still owed)
#pragma unroll
            for (int m = 0; m < 4; ++m) { Gj[m][0] *= f; Gj[m][1] *= f; Gj[m][2] *= f; Gj[m][3] *= f; }
            if (keep_operand) {
                GmL = acc_as_operand(Gj[0], Gj[1]); GmH = acc_as_operand(Gj[2], Gj[3]);
                // also for the gv role of the producer waves: row j = col, value channels 8g .. 8g+7 and 32 + 8g .. +7
                unsigned char *gt = smem + BlockBwdLds::kGt + blk * kTileBytes;
                *reinterpret_cast<bf16x8 *>(gt + gt_lo) = GmL;
                *reinterpret_cast<bf16x8 *>(gt + gt_hi) = GmH;
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0) g_flags[4 * blk + q] = it + 1;
            }
            s16x4 gq[2][4], rtq[2];
#pragma unroll
            for (int pp = 0; pp < 2; ++pp) {
                rtq[pp] = la.frag_tok(rt, q, 32 * blk + 16 * pp);
#pragma unroll
                for (int m = 0; m < 4; ++m) gq[pp][m] = la.frag_tok_rows(gyt, m, 32 * blk + 16 * pp);
            }
#pragma unroll
            for (int pp = 0; pp < 2; ++pp)
#pragma unroll
                for (int m = 0; m < 4; ++m) Gj[m] = mfma16(gq[pp][m], rtq[pp], Gj[m]);
            settle(Gj[0], Gj[1], Gj[2], Gj[3]);
            pend = g1c;
        };
        // E[j = col] = sum_i S[j][i] G[j][i] with S as fp32 values in the layout of Gj; then to the lanes that hold channel col as a row
        float pre[4];
        auto anchor = [&](const f32x4 (&Sv)[4]) {
            float e0 = 0.f, e1 = 0.f;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                e0 = fmaf(Sv[m][0], Gj[m][0], e0); e1 = fmaf(Sv[m][1], Gj[m][1], e1);
                e0 = fmaf(Sv[m][2], Gj[m][2], e0); e1 = fmaf(Sv[m][3], Gj[m][3], e1);
            }
            const float E = sum_rows((e0 + e1) * pend);
            if (g == 0) scratch[l16] = E;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // (one wave: its LDS accesses are executed in order)
            const float4 E4 = *reinterpret_cast<const float4 *>(&scratch[4 * g]);
            pre[0] = E4.x; pre[1] = E4.y; pre[2] = E4.z; pre[3] = E4.w;
        };
        f32x4 Sv[4];
#pragma unroll
        for (int m = 0; m < 4; ++m)
            Sv[m] = (f32x4){__uint_as_float(Sraw[m][0] << 16), __uint_as_float(Sraw[m][0] & 0xffff0000u),
                            __uint_as_float(Sraw[m][1] << 16), __uint_as_float(Sraw[m][1] & 0xffff0000u)};
        bf16x8 sL, sH;
        if (HALF == 1) {
            // the later block: G arrives at its end; its S is the saved state stepped over the earlier block
            step_G(1, g1c1, g2c1, true);
            {
                s16x4 vq[2][4], ktq[2];
#pragma unroll
                for (int pp = 0; pp < 2; ++pp) {
                    ktq[pp] = la.frag_tok(kt, q, 16 * pp);
#pragma unroll
                    for (int m = 0; m < 4; ++m) vq[pp][m] = la.frag_tok_rows(vt, m, 16 * pp);
                }
#pragma unroll
                for (int m = 0; m < 4; ++m) { Sv[m][0] *= g1c0; Sv[m][1] *= g1c0; Sv[m][2] *= g1c0; Sv[m][3] *= g1c0; }
#pragma unroll
                for (int pp = 0; pp < 2; ++pp)
#pragma unroll
                    for (int m = 0; m < 4; ++m) Sv[m] = mfma16(vq[pp][m], ktq[pp], Sv[m]);
                settle(Sv[0], Sv[1], Sv[2], Sv[3]);
#pragma unroll
                for (int m = 0; m < 4; ++m) { Sv[m][0] *= g2c0; Sv[m][1] *= g2c0; Sv[m][2] *= g2c0; Sv[m][3] *= g2c0; }
            }
            sL = acc_as_operand(Sv[0], Sv[1]); sH = acc_as_operand(Sv[2], Sv[3]);
            // (the anchor takes S as X does, rounded to bf16: the flow balance holds between what X, W and E see)
            {
                float lo[8], hi[8];
                unpack8(sL, lo); unpack8(sH, hi);
#pragma unroll
                for (int e = 0; e < 4; ++e) { Sv[0][e] = lo[e]; Sv[1][e] = lo[4 + e]; Sv[2][e] = hi[e]; Sv[3][e] = hi[4 + e]; }
            }
            anchor(Sv);
            step_G(0, g1c0, g2c0, false);   // on to the chunk start (what the next visit continues from)
        } else {
            // the earlier block: G has to cross the later block first; its S is the saved state
            step_G(1, g1c1, g2c1, false);
            step_G(0, g1c0, g2c0, true);
            sL = make_bf16x8(Sraw[0][0], Sraw[0][1], Sraw[1][0], Sraw[1][1]);
            sH = make_bf16x8(Sraw[2][0], Sraw[2][1], Sraw[3][0], Sraw[3][1]);
            anchor(Sv);
        }
        // This block's two 16-token row groups (p0 first): fragments of gy, v with the k-slots along the value channels
        constexpr int P0 = 2 * HALF;
        constexpr int R0 = 16 * P0, R1 = R0 + 16;   // first rows of the two groups
        f32x4 X0[2], X1[2], W0[2], W1[2];
        float vg[2];
        {
            const s16x4 kq0 = la.frag_tok(kt, q, R0), kq1 = la.frag_tok(kt, q, R1);
            const s16x4 rq0 = la.frag_tok(rt, q, R0), rq1 = la.frag_tok(rt, q, R1);
            // state terms X0, W0 (rows j = 4g + rr of this wave's 16 channels, column = token l16);
            // dA^T (rows s, column t): blocks (0,0), (0,1), (1,1);  dA (rows t, column s): blocks (0,0), (1,0), (1,1).
            // The value channels are covered in two halves of 32, so that only one half's fragments are live.
            f32x4 T00, T01, T11, D00, D10, D11;
            {
                const bf16x8 gf0 = la.frag_ch(gyt, R0, 0), gf1 = la.frag_ch(gyt, R1, 0);
                const bf16x8 vf0 = la.frag_ch(vt, R0, 0), vf1 = la.frag_ch(vt, R1, 0);
                X0[0] = mfma32(sL, gf0, zero); X0[1] = mfma32(sL, gf1, zero);
                W0[0] = mfma32(GmL, vf0, zero); W0[1] = mfma32(GmL, vf1, zero);
                T00 = mfma32(vf0, gf0, zero); T01 = mfma32(vf0, gf1, zero); T11 = mfma32(vf1, gf1, zero);
                D00 = mfma32(gf0, vf0, zero); D10 = mfma32(gf1, vf0, zero); D11 = mfma32(gf1, vf1, zero);
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                const bf16x8 gf0 = la.frag_ch(gyt, R0, 1), gf1 = la.frag_ch(gyt, R1, 1);
                const bf16x8 vf0 = la.frag_ch(vt, R0, 1), vf1 = la.frag_ch(vt, R1, 1);
                X0[0] = mfma32(sH, gf0, X0[0]); X0[1] = mfma32(sH, gf1, X0[1]);
                W0[0] = mfma32(GmH, vf0, W0[0]); W0[1] = mfma32(GmH, vf1, W0[1]);
                T00 = mfma32(vf0, gf0, T00); T01 = mfma32(vf0, gf1, T01); T11 = mfma32(vf1, gf1, T11);
                D00 = mfma32(gf0, vf0, D00); D10 = mfma32(gf1, vf0, D10); D11 = mfma32(gf1, vf1, D11);
            }
            settle(T00, T01, T11);
            settle(D00, D10, D11);
            // the diagonal of dA is <v_t, gy_t>: picked out of the lanes that hold it, then shared over the four rows
            {
                const bool odd = l16 & 1, hi = l16 & 2, mine = (l16 >> 2) == g;
                const float a01 = odd ? D00[1] : D00[0], a23 = odd ? D00[3] : D00[2];
                const float b01 = odd ? D11[1] : D11[0], b23 = odd ? D11[3] : D11[2];
                vg[0] = sum_rows(mine ? (hi ? a23 : a01) : 0.f);
                vg[1] = sum_rows(mine ? (hi ? b23 : b01) : 0.f);
            }
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int x = 4 * g + rr;
                D00[rr] = (x > l16) ? D00[rr] : 0.f; D11[rr] = (x > l16) ? D11[rr] : 0.f;      // rows t, column s: t > s
                T00[rr] = (l16 > x) ? T00[rr] : 0.f; T11[rr] = (l16 > x) ? T11[rr] : 0.f;      // rows s, column t: t > s
            }
            X1[0] = mfma16(kq0, pack4(T00), zero);
            X1[1] = mfma16(kq0, pack4(T01), zero);
            W1[0] = mfma16(rq0, pack4(D00), zero);
            W1[1] = mfma16(rq1, pack4(D11), zero);
            X1[1] = mfma16(kq1, pack4(T11), X1[1]);
            W1[0] = mfma16(rq1, pack4(D10), W1[0]);
        }
        settle(X0[0], X0[1], W0[0], W0[1]);
        settle(X1[0], X1[1], W1[0], W1[1]);
        // elementwise pass: lane (l16, g) <-> token of row group n, channels 16q + 4g + rr
        const float g1s[4] = {g1r.x, g1r.y, g1r.z, g1r.w};
        uint32_t packed[3][2][2];   // [gr, gk, gw][row group][channel pair]
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const uint32_t o = la_cols + (uint32_t)((n == 0 ? R0 : R1) * kTileRow);
            float rt_[4], kt_[4], an[4], ew[4];
            {
                const uint2 xr = *reinterpret_cast<const uint2 *>(rt + o), xk = *reinterpret_cast<const uint2 *>(kt + o);
                const uint2 xa = *reinterpret_cast<const uint2 *>(at + o), xw = *reinterpret_cast<const uint2 *>(wt + o);
                unpack4(make_s16x4(xr.x, xr.y), rt_); unpack4(make_s16x4(xk.x, xk.y), kt_);
                unpack4(make_s16x4(xa.x, xa.y), an); unpack4(make_s16x4(xw.x, xw.y), ew);
            }
            float gro[4], gko[4], gwo[4], D[4], Pv[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                // alpha_t is the previous token's alpha_{t+1} (the lane before); the block's first token has
                // 1 / g1, its middle token (the second group's first) exactly 1
                const float a_n = an[rr], ia_n = __builtin_amdgcn_rcpf(a_n);
                const float a_t = prev_in_row16(a_n, n == 0 ? __builtin_amdgcn_rcpf(g1s[rr]) : 1.f);
                const float ia_t = prev_in_row16(ia_n, n == 0 ? g1s[rr] : 1.f);
                const float X = fmaf(g1s[rr], X0[n][rr], X1[n][rr]);
                const float W = W0[n][rr] + W1[n][rr];
                const float rraw = rt_[rr] * ia_t, kraw = kt_[rr] * a_n;
                const float uvg = u4[rr] * vg[n];
                Pv[rr] = rt_[rr] * X;
                D[rr] = fmaf(kt_[rr], W, -Pv[rr]);
                gro[rr] = fmaf(a_t, X, uvg * kraw);
                gko[rr] = fmaf(ia_n, W, uvg * rraw);
                gu_acc[rr] = fmaf(rraw * kraw, vg[n], gu_acc[rr]);
            }
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const float incl = scan_row16(D[rr]);
                gwo[rr] = -ew[rr] * (pre[rr] + (incl - D[rr]) - Pv[rr]);
                pre[rr] += last_of_row16(incl);
            }
            // the gradient of the first and the last decay of the sequence is zero by definition (the flow
            // balance leaves rounding residue there)
            // (with an initial state / a gradient arriving at the final state they are not zero)
            if ((HALF == 0 && n == 0 && c == 0 && l16 == 0 && !has_s0) ||
                ((kRagged ? c * kBlockTokens + (n == 0 ? R0 : R1) + l16 == T - 1 : (HALF == 1 && n == 1 && c == nchunk - 1 && l16 == 15)) && !gsT)) {
                gwo[0] = gwo[1] = gwo[2] = gwo[3] = 0.f;
            }
            packed[0][n][0] = pack_bf16x2(gro[0], gro[1]); packed[0][n][1] = pack_bf16x2(gro[2], gro[3]);
            packed[1][n][0] = pack_bf16x2(gko[0], gko[1]); packed[1][n][1] = pack_bf16x2(gko[2], gko[3]);
            packed[2][n][0] = pack_bf16x2(gwo[0], gwo[1]); packed[2][n][1] = pack_bf16x2(gwo[2], gwo[3]);
        }
        {
            // 16 bytes per lane: token (g odd ? R1 : R0) + l16, channels 16q + 8 (g >> 1) .. +7
            const int tok = c * kBlockTokens + R0 + 16 * (g & 1) + l16;
            const uint32_t go = (uint32_t)tok * rowbytes + 2u * (uint32_t)(16 * q + 8 * (g >> 1));
            const u32x4 o_r = pair_rows_8ch(packed[0][0][0], packed[0][0][1], packed[0][1][0], packed[0][1][1]);
            const u32x4 o_k = pair_rows_8ch(packed[1][0][0], packed[1][0][1], packed[1][1][0], packed[1][1][1]);
            const u32x4 o_w = pair_rows_8ch(packed[2][0][0], packed[2][0][1], packed[2][1][0], packed[2][1][1]);
            if (!kRagged || tok < T) {   // (rows past the end of the sequence are not written)
                *reinterpret_cast<u32x4 *>(gr_h + go) = o_r;
                *reinterpret_cast<u32x4 *>(gk_h + go) = o_k;
                *reinterpret_cast<u32x4 *>(gw_h + go) = o_w;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (++cv == nchunk) {
            // the pair is done.  The reverse state has arrived at t = 0: dL/dS_0 (both halves hold it)
            if (gs0 && HALF == 0) {
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    *reinterpret_cast<f32x4 *>(gs0 + (int64_t)((b0 + slot * a.bstep) * H + h) * (kN * kN) + col * kN + block_row_channel(m, g)) =
                        (f32x4){Gj[m][0] * pend, Gj[m][1] * pend, Gj[m][2] * pend, Gj[m][3] * pend};
            }
            // gu: fold the 16 tokens of a row; lanes l16 = 0 hold channels 16q + 4g + rr
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) gu_acc[rr] = sum_row16(gu_acc[rr]);
            if (l16 == 0) *reinterpret_cast<float4 *>(&gu_lds[((slot & 1) * 2 + HALF) * kN + 16 * q + 4 * g]) = make_float4(gu_acc[0], gu_acc[1], gu_acc[2], gu_acc[3]);
            cv = 0;
            ++slot;
        }
    }
    __threadfence_block();
    __syncthreads();
    if (HALF == 0) deliver_gu(npw - 1);
}

// ------------------------------------------------------------------------------------------
// gv role of a producer wave: wave q owns value columns i = 16q..16q+15.  The reverse state comes from
// the waves that step it (g2 o G at the end of each block, as they publish it in kGt).
// ------------------------------------------------------------------------------------------
template <bool kRagged>
__device__ __forceinline__ void block_bwd_gv(const unsigned char *smem, bf16_t *gv_h, uint32_t rowelems, int T, int c, int it, int q, int lane)
{
    const int g = lane >> 4, l16 = lane & 15;
    const unsigned char *rt = smem + BlockBwdLds::kRawRK + (it % 3) * 2 * kTileBytes, *kt = rt + kTileBytes;
    const unsigned char *gyt = smem + BlockBwdLds::kRawVG + (it & 1) * 2 * kTileBytes + kTileBytes;
    const float *vec = reinterpret_cast<const float *>(smem + BlockBwdLds::kVec + (it & 1) * kBlockVecBytes), *ruk = vec + 4 * kN;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const BlockLane la(l16, g);
    // operand fragment G[j = 32h + 8g + e][i = 16q + l16], e < 8, out of the [j][i] tile: two transposing reads of
    // four rows each (rows 8g + (l16 >> 2) and four further on, the lane's 8-byte piece of channels 16q + 4 (l16 & 3) ..)
    const uint32_t gt_a = ((uint32_t)(8 * g + (l16 >> 2)) << 7) + ((((uint32_t)(2 * q) | (((uint32_t)l16 >> 1) & 1u)) ^ ((uint32_t)l16 >> 2)) << 4) + (((uint32_t)l16 & 1u) << 3);
    const uint32_t gt_b = (gt_a ^ 64u) + 4 * kTileRow;
    LdsFlag g_flags = (LdsFlag)(smem + BlockBwdLds::kGFlags);
#pragma unroll
    for (int blk = 1; blk >= 0; --blk) {
        while (g_flags[4 * blk] < it + 1 || g_flags[4 * blk + 1] < it + 1 || g_flags[4 * blk + 2] < it + 1 || g_flags[4 * blk + 3] < it + 1)
            __builtin_amdgcn_s_sleep(1);
        const unsigned char *gt = smem + BlockBwdLds::kGt + blk * kTileBytes;
        auto g_frag = [&](int h) {
            const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(gt + gt_a + h * 32 * kTileRow)));
            const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(gt + gt_b + h * 32 * kTileRow)));
            return make_bf16x8(lo[0], lo[1], hi[0], hi[1]);
        };
        const bf16x8 GmL = g_frag(0), GmH = g_frag(1);
        const int R0 = 32 * blk, R1 = R0 + 16, r0 = R0 + l16, r1 = R1 + l16;
        const s16x4 gyq0 = la.frag_tok(gyt, q, R0), gyq1 = la.frag_tok(gyt, q, R1);
        const float ruk0 = ruk[r0], ruk1 = ruk[r1];
        // products transposed: accumulator rows i = 4g + rr, column s = l16.  A[t][s] (rows t = 4g + rr, column s):
        // blocks (0,0), (1,0), (1,1).  The key channels are covered in two halves of 32 (one half's fragments live).
        f32x4 GV0, GV1, A00, A10, A11;
        {
            const bf16x8 rf0 = la.frag_ch(rt, R0, 0), rf1 = la.frag_ch(rt, R1, 0);
            const bf16x8 kf0 = la.frag_ch(kt, R0, 0), kf1 = la.frag_ch(kt, R1, 0);
            GV0 = mfma32(GmL, kf0, zero); GV1 = mfma32(GmL, kf1, zero);
            A00 = mfma32(rf0, kf0, zero); A10 = mfma32(rf1, kf0, zero); A11 = mfma32(rf1, kf1, zero);
        }
        __builtin_amdgcn_sched_barrier(0);
        {
            const bf16x8 rf0 = la.frag_ch(rt, R0, 1), rf1 = la.frag_ch(rt, R1, 1);
            const bf16x8 kf0 = la.frag_ch(kt, R0, 1), kf1 = la.frag_ch(kt, R1, 1);
            GV0 = mfma32(GmH, kf0, GV0); GV1 = mfma32(GmH, kf1, GV1);
            A00 = mfma32(rf0, kf0, A00); A10 = mfma32(rf1, kf0, A10); A11 = mfma32(rf1, kf1, A11);
        }
        __builtin_amdgcn_sched_barrier(0);
        settle(A00, A10, A11);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int x = 4 * g + rr;
            A00[rr] = (x > l16) ? A00[rr] : ((x == l16) ? ruk0 : 0.f);
            A11[rr] = (x > l16) ? A11[rr] : ((x == l16) ? ruk1 : 0.f);
        }
        f32x4 V0 = mfma16(gyq0, pack4(A00), zero), V1 = mfma16(gyq1, pack4(A11), zero);
        V0 = mfma16(gyq1, pack4(A10), V0);
        settle(GV0, GV1, V0, V1);
        // 16 bytes per lane: token (g odd ? R1 : R0) + l16, channels 16q + 8 (g >> 1) .. +7
        const int tok = c * kBlockTokens + R0 + 16 * (g & 1) + l16;
        const u32x4 o_v = pair_rows_8ch(pack_bf16x2(GV0[0] + V0[0], GV0[1] + V0[1]), pack_bf16x2(GV0[2] + V0[2], GV0[3] + V0[3]),
                                        pack_bf16x2(GV1[0] + V1[0], GV1[1] + V1[1]), pack_bf16x2(GV1[2] + V1[2], GV1[3] + V1[3]));
        if (!kRagged || tok < T) *reinterpret_cast<u32x4 *>(gv_h + ((uint32_t)tok * rowelems + (uint32_t)(16 * q + 8 * (g >> 1)))) = o_v;
    }
}

// ------------------------------------------------------------------------------------------
// Producer wave p: loads, operand preparation of tokens 16p..16p+15, then the gv role.
// ------------------------------------------------------------------------------------------
template <bool kMulti, bool kRagged>
__device__ __forceinline__ void block_bwd_producer(const BlockBwdArgs &a, unsigned char *smem, int *s_wild, int pair0, int p, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + kBlockTokens - 1) / kBlockTokens;
    const int b0 = pair0 / H, h = pair0 - b0 * H;
    const int npw = kMulti ? (a.B - b0 + a.bstep - 1) / a.bstep : 1;
    const int nvisit = npw * nchunk;
    const uint32_t rowbytes = (uint32_t)C * 2u;
    const uint32_t lds0 = lds_address(smem);
    // first element of the workgroup's pair number `slot` in a (B,T,C) tensor; its saved states
    auto pair_base = [&](int slot) { return (int64_t)(b0 + slot * a.bstep) * T * C + (int64_t)h * kN; };
    auto pair_states = [&](int slot) {
        return reinterpret_cast<const bf16_t *>(a.ckpt + (int64_t)((b0 + slot * a.bstep) * H + h) * nchunk * (kN * kN));
    };
    const int lrow = lane >> 3;
    const uint32_t lpiece = (uint32_t)(((lane & 7) ^ lrow) << 4);
    // byte offset of this lane's piece of token row t of a pair (kRagged: rows past the end read the last row)
    auto row_offset = [&](int t) { return (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + lpiece; };
    // Every stream walks the flat sequence of visits (pair 0 chunk nchunk-1, .., 0, pair 1 chunk nchunk-1, ..) with
    // a cursor of its own: visit number `it`, its position `c` in its pair (chunk nchunk-1-c), the pair's number.
    struct Cursor {
        int it = 0, c = 0, slot = 0;
    };
    Cursor cr, cg, cp, co;   // r/k/w loads, v/gy/state loads, operand preparation, gv role
    const bf16_t *rb = a.r + pair_base(0), *kb_ = a.k + pair_base(0), *wb = a.w + pair_base(0);
    const bf16_t *vb = a.v + pair_base(0), *gb = a.gy + pair_base(0), *ckb = pair_states(0);
    bf16_t *gvb = a.gv + pair_base(0);
    // r, k, w go out two visits ahead (they are prepared one visit ahead), v, gy and the chunk's saved state one
    // visit ahead.
    auto issue_rkw = [&]() {
        const int tb = (nchunk - 1 - cr.c) * kBlockTokens + 16 * p;
        const uint32_t rk = lds0 + BlockBwdLds::kRawRK + (cr.it % 3) * 2 * kTileBytes + 16 * p * kTileRow;
        const uint32_t ww = lds0 + BlockBwdLds::kRawW + (cr.it % 3) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const uint32_t o = row_offset(tb + 8 * hf + lrow);
            load_rows8_to_lds(kb_, o, rk + kTileBytes + 8 * hf * kTileRow);
            load_rows8_to_lds(wb, o, ww + 8 * hf * kTileRow);
            load_rows8_to_lds(rb, o, rk + 8 * hf * kTileRow);
        }
        ++cr.it;
        if (kMulti && ++cr.c == nchunk) {
            cr.c = 0; ++cr.slot;
            const int64_t nb = pair_base(cr.slot);
            rb = a.r + nb; kb_ = a.k + nb; wb = a.w + nb;
        } else if (!kMulti) ++cr.c;
    };
    auto issue_vg_state = [&]() {
        const int tb = (nchunk - 1 - cg.c) * kBlockTokens + 16 * p;
        const uint32_t vg = lds0 + BlockBwdLds::kRawVG + (cg.it & 1) * 2 * kTileBytes + 16 * p * kTileRow;
        const bf16_t *src = ckb + (int64_t)(nchunk - 1 - cg.c) * (kN * kN);
        const uint32_t dst = lds0 + BlockBwdLds::kState + (cg.it & 1) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const uint32_t o = row_offset(tb + 8 * hf + lrow);
            load_rows8_to_lds(src, (uint32_t)((16 * p + 8 * hf + lrow) * kTileRow) + lpiece, dst + 8 * hf * kTileRow);
            load_rows8_to_lds(vb, o, vg + 8 * hf * kTileRow);
            load_rows8_to_lds(gb, o, vg + kTileBytes + 8 * hf * kTileRow);
        }
        ++cg.it;
        if (kMulti && ++cg.c == nchunk) {
            cg.c = 0; ++cg.slot;
            const int64_t nb = pair_base(cg.slot);
            vb = a.v + nb; gb = a.gy + nb; ckb = pair_states(cg.slot);
        } else if (!kMulti) ++cg.c;
    };
    float u4[4];
    load4(a.u + h * kN + 4 * l16, u4);   // (all pairs of a workgroup belong to one head)
    // the next visit in line; `younger`: vector-memory operations this wave has issued behind that visit's tile
    // loads (a wave's operations complete in program order, so those may stay in flight)
    auto prepare = [&](int younger) {
        const int it = cp.it;
        unsigned char *rk = smem + BlockBwdLds::kRawRK + (it % 3) * 2 * kTileBytes;
        unsigned char *ww = smem + BlockBwdLds::kRawW + (it % 3) * kTileBytes;
        unsigned char *al = smem + BlockBwdLds::kAlpha + (it & 1) * kTileBytes;
        float *vec = reinterpret_cast<float *>(smem + BlockBwdLds::kVec + (it & 1) * kBlockVecBytes);
        wait_in_flight(younger);
        const float kLn2 = 0.6931471805599453f;
        const bool ok = block_prepare<kRagged>(rk, rk + kTileBytes, ww, vec, u4, p, l16, g, T - (nchunk - 1 - cp.c) * kBlockTokens, []() {},
            [&](uint32_t o, const float (&xr)[4], const float (&xk)[4], const float (&xa)[4], const float (&ew2)[4]) {
                // R~ and K~ take the place of the raw r and k, exp(w) that of the raw w
                *reinterpret_cast<uint2 *>(rk + o) = make_uint2(pack_bf16x2(xr[0], xr[1]), pack_bf16x2(xr[2], xr[3]));
                *reinterpret_cast<uint2 *>(rk + kTileBytes + o) = make_uint2(pack_bf16x2(xk[0], xk[1]), pack_bf16x2(xk[2], xk[3]));
                *reinterpret_cast<uint2 *>(al + o) = make_uint2(pack_bf16x2(xa[0], xa[1]), pack_bf16x2(xa[2], xa[3]));
                *reinterpret_cast<uint2 *>(ww + o) = make_uint2(pack_bf16x2(ew2[0] * kLn2, ew2[1] * kLn2), pack_bf16x2(ew2[2] * kLn2, ew2[3] * kLn2));
            });
        if (!ok && lane == 0) s_wild[cp.slot] = 1;
        ++cp.it;
        ++cp.c;
        if (kMulti && cp.c == nchunk) { cp.c = 0; ++cp.slot; }
    };
    constexpr int kRkwLoads = 6, kVgStateLoads = 6;
    // gv stores a visit leaves in flight.  The chunk with the ragged end issues anything from 0 to 2 (a store
    // whose lanes are all past the end is skipped): counting none for it makes the waits behind it wait for
    // everything older, whereas counting one that was not issued would let them return early.
    auto gv_stores = [&](int pos) { return (kRagged && pos == 0) ? 0 : 2; };   // pos: the visit's position in its pair
    int gv_before = 0;   // of the visit before
    issue_vg_state();
    issue_rkw();
    if (nvisit > 1) issue_rkw();
    prepare(nvisit > 1 ? kRkwLoads : 0);
    for (int it = 0; it < nvisit; ++it) {
        __syncthreads();
        // free again: every tile of visit it-1
        const int vgs = it + 1 < nvisit ? kVgStateLoads : 0, rkw = it + 2 < nvisit ? kRkwLoads : 0;
        if (it + 1 < nvisit) issue_vg_state();
        if (it + 2 < nvisit) issue_rkw();
        // behind the r, k, w loads of visit it+1 (issued one visit ago): that visit's gv stores, and this visit's loads
        if (it + 1 < nvisit) prepare(gv_before + vgs + rkw);
        block_bwd_gv<kRagged>(smem, gvb, (uint32_t)C, T, nchunk - 1 - co.c, it, p, lane);
        gv_before = gv_stores(co.c);
        ++co.c;
        if (kMulti && co.c == nchunk) { co.c = 0; ++co.slot; gvb = a.gv + pair_base(co.slot); }
        // v, gy and the state of the next visit have to be in LDS when the other waves pass the barrier
        if (it + 1 < nvisit) wait_in_flight(rkw + gv_before);
    }
    wait_loads<0>();
    __threadfence_block();
    __syncthreads();
}

constexpr int kBlockBwdThreads = 12 * 64;

template <bool kMulti, bool kRagged>   // kMulti: a workgroup takes several pairs, one after the other; kRagged: T is no multiple of 64
__global__ __launch_bounds__(kBlockBwdThreads) void block_bwd_kernel(BlockBwdArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild[kBlockMaxSlots];   // per pair of the workgroup: 16 tokens left the scaled operands' range
    __shared__ float s_ft[kN];               // exact second pass with state gradients: the anchor of the gw sums
    static_assert(sizeof(ScanBwdALds) <= BlockBwdLds::kBytes && sizeof(ScanBwdBLds) <= BlockBwdLds::kBytes,
                  "the exact second pass reuses the LDS block");
    if (threadIdx.x < kBlockMaxSlots) s_wild[threadIdx.x] = 0;
    if (threadIdx.x < 8) reinterpret_cast<int *>(smem + BlockBwdLds::kGFlags)[threadIdx.x] = 0;
    __syncthreads();

    const int pair0 = (int)blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave < 4) block_bwd_producer<kMulti, kRagged>(a, smem, s_wild, pair0, wave, lane);
    else if (wave < 8) block_bwd_xw<0, kMulti, kRagged>(a, smem, s_wild, pair0, wave - 4, lane);
    else block_bwd_xw<1, kMulti, kRagged>(a, smem, s_wild, pair0, wave - 8, lane);
    const int b0 = pair0 / a.H, h = pair0 - b0 * a.H;
    const int npw = kMulti ? (a.B - b0 + a.bstep - 1) / a.bstep : 1;
    const int nchunk = (a.T + kBlockTokens - 1) / kBlockTokens;
    const int64_t slice = (int64_t)nchunk * (kN * kN), C = (int64_t)a.H * kN;
    const int tid = threadIdx.x;
    __threadfence_block();
    __syncthreads();
    // gu summed over the workgroup's pairs that the chunked code did (half 0 added them up as it stored them): out
    // of the way of the second pass, which uses the whole LDS block
    __shared__ float s_gu_wg[kN];
    if (tid < kN) s_gu_wg[tid] = reinterpret_cast<const float *>(smem + BlockBwdLds::kGu)[4 * kN + tid];
    // exact second pass for the pairs of which 16 tokens left the range the scaled operands can hold; the
    // pair's own slice of the state workspace (nchunk x 64 x 64 floats = T x 64) holds P
    for (int slot = 0; slot < npw; ++slot) {
        if (!s_wild[slot]) continue;   // (uniform over the workgroup)
        const int b = b0 + slot * a.bstep;
        // (the pointers pass through a value the compiler cannot see through, so that nothing derived from them is
        // computed ahead of the loop and kept in registers across the chunked code)
        const int z = fresh_s(0);
        float *ck = a.ckpt + (int64_t)(b * a.H + h) * slice + z;
        const int64_t so = (int64_t)(b * a.H + h) * (kN * kN) + z;
        const float *s0p = !kMulti && a.s0 ? a.s0 + so : nullptr, *gsTp = !kMulti && a.gsT ? a.gsT + so : nullptr;
        float *gs0p = !kMulti && a.gs0 ? a.gs0 + so : nullptr;
        const bool states = s0p || gsTp || gs0p;
        __syncthreads();
        scan_bwd_a_body<bf16_t, bf16_t>(*reinterpret_cast<ScanBwdALds *>(smem), b, h, a.T, a.H, a.r + z, a.k + z, a.v + z, a.w + z, a.u + z, a.gy + z,
                                        a.gr + z, a.gu + z, ck, kN, s0p, gsTp, states ? s_ft : nullptr);
        __threadfence_block();
        __syncthreads();
        const int z2 = fresh_s(0);
        scan_bwd_b_body<bf16_t, bf16_t>(*reinterpret_cast<ScanBwdBLds *>(smem), b, h, a.T, a.H, a.r + z2, a.k + z2, a.v + z2, a.w + z2, a.u + z2, a.gy + z2,
                                        ck + z2, kN, a.gk + z2, a.gv + z2, a.gw + z2, gsTp, states ? s_ft : nullptr, gs0p, s0p == nullptr);
        __threadfence_block();
        __syncthreads();
    }
    // (addresses formed from here on are not to be computed ahead of the second pass and kept across it)
    int lane_id = tid;
    asm volatile("" : "+v"(lane_id));
    float part = 0.f;
    if (a.gu_sum != nullptr && lane_id < kN) {
        part = s_gu_wg[lane_id];
        for (int slot = 0; slot < npw; ++slot)   // the redone pairs' rows, as the second pass stored them
            if (s_wild[slot]) part += load1(a.gu + (int64_t)(b0 + slot * a.bstep) * C + h * kN + lane_id);
    }
    // Fused batch sum of gu: the workgroup that is the last of its head to deliver adds up the partials, one per
    // workgroup of the head.  They travel as written-through (agent scope) stores into the unused second half of
    // the workspace slice of each workgroup's first pair, completed before the arrival counter is bumped; no
    // fence, which would write back the whole L2.
    if (a.gu_sum != nullptr) {
        __shared__ int s_last;
        const int nparts = a.bstep;   // workgroups of this head (first pairs h, h + H, ..)
        if (tid < kN) {          // wave 0
            __hip_atomic_store(a.ckpt + (int64_t)pair0 * slice + slice / 2 + lane_id, part, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (tid == 0)
                s_last = __hip_atomic_fetch_add(a.arrivals + h, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nparts - 1;
        }
        __syncthreads();
        if (s_last && tid < kN) {
            float acc = 0.f;
            for (int j = 0; j < nparts; ++j)
                acc += __hip_atomic_load(a.ckpt + (int64_t)(h + j * a.H) * slice + slice / 2 + lane_id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            store1(a.gu_sum + h * kN + lane_id, acc);
            if (tid == 0) __hip_atomic_store(a.arrivals + h, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // armed again
        }
    }
}

bool block_backward_applies(int64_t B, int64_t T, int64_t H) { return block_forward_applies(B, T, H); }

hipError_t block_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, void *gu_sum,
                          const float *s0, const float *gsT, float *gs0)
{
    BlockBwdArgs a = {};
    a.T = (int)T; a.H = (int)H; a.B = (int)B;
    const int64_t grid = block_grid(B, H);
    a.bstep = B * H <= grid ? (int)B : (int)(grid / H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w;
    a.u = (const bf16_t *)u; a.gy = (const bf16_t *)gy;
    a.gr = (bf16_t *)gr; a.gk = (bf16_t *)gk; a.gv = (bf16_t *)gv; a.gw = (bf16_t *)gw; a.gu = (bf16_t *)gu;
    a.gu_sum = (bf16_t *)gu_sum;
    a.s0 = s0; a.gsT = gsT; a.gs0 = gs0;
    a.ckpt = (float *)workspace;
    a.arrivals = reinterpret_cast<int *>(reinterpret_cast<char *>(workspace) + chunk_backward_workspace_bytes(B, T, H));
    const bool multi = B * H > grid, ragged = (T % kBlockTokens) != 0;
    auto launch = [&](auto multi_tag, auto ragged_tag) -> hipError_t {
        constexpr auto kern = block_bwd_kernel<decltype(multi_tag)::value, decltype(ragged_tag)::value>;
        hipError_t e = allow_dynamic_lds<kern>(BlockBwdLds::kBytes);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kBlockBwdThreads), BlockBwdLds::kBytes, st, a);
        return hipGetLastError();
    };
    if (multi) return ragged ? launch(std::true_type{}, std::true_type{}) : launch(std::true_type{}, std::false_type{});
    return ragged ? launch(std::false_type{}, std::true_type{}) : launch(std::false_type{}, std::false_type{});
}

}  // namespace wkv6
