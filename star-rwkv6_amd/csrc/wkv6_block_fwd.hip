// WKV6 forward in block form for gfx950 (bf16 MFMA for the dense products, fp32 state), for bf16
// tensors and more than half a (batch, head) pair per compute unit (a sequence length that is no
// multiple of 64 leaves the last chunk with tokens past the end: kRagged).  The tile form in wkv6_chunk_fwd.hip (state advanced every 16 tokens) serves every
// other case.  Notation and the operand scaling are in wkv6_block.h.
//
// One workgroup per pair; with more pairs than compute units one workgroup per compute unit, which runs
// its pairs (same head, `bstep` batch rows apart) back to back through ONE pipeline: the loads, the
// operand preparation and the stores each walk the flat sequence of (pair, chunk) visits with a cursor
// of their own, so a pair's first chunks are loaded and prepared while the pair before it finishes.
//
// Per block of 32 tokens (S = state entering it, rows j):
//   A[t][s] = R~_t . K~_s (s < t),   A[t][t] = sum_j r_t[j] u[j] k_t[j]
//   Y  = R~ (g1 o S) + A V
//   S <- g2 o (g1 o S + K~^T V)
// The state is touched twice per block (two scalings and one MFMA accumulation over its 32 tokens)
// instead of once per 16-token tile; A is three 16x16 blocks; nothing but the scalings and the masks
// of the diagonal blocks is VALU work in the consumer waves.
//
// Workgroup: 12 waves in three roles, one wave of each per SIMD.  Four loading waves (wave p <-> tokens
// 16p..16p+15 of every chunk) bring the raw rows from global memory straight into LDS three chunk visits
// ahead and turn r, k, w of the next chunk into R~, K~, g1, g2 and the diagonal.  Four consumer waves
// (q): value columns 16q..16q+15 of the state and of y, both blocks of a visit.  Four storing waves
// write out what the consumers staged during the previous visit (kFuse: with the output stage, whose
// gate rows they fetch themselves): y and the saved chunk states never leave a consumer wave as partial
// rows, they are staged in LDS as [token][channel] tiles and leave one visit later as whole 128-byte rows.
// (Loads and stores in different waves: a wave's vector-memory operations complete in order, and a
// loading wave that also stored waited for its stores with every load; two sets of consumer waves that
// both carried the state took as long as one.)
#include "wkv6_mfma.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"
#include "wkv6_block.h"

#include <type_traits>

namespace wkv6 {

// kFuse (the output stage in the kernel): the gate's rows come in like v, one visit before they are used, and v
// is requested two visits ahead instead of three to make room for them.
template <bool kFuse>
struct BlockFwdLdsT {
    static constexpr int kVAhead = kFuse ? 2 : 3;                        // visits between the request of v and its use
    static constexpr int kRaw = 0;                                       // [2 visit parities][r, k, w] raw tiles
    static constexpr int kRawV = kRaw + 2 * 3 * kTileBytes;              // [visit % (kVAhead + 1)] raw v tiles
    static constexpr int kOp = kRawV + (kVAhead + 1) * kTileBytes;       // [2][R~, K~]
    static constexpr int kVec = kOp + 2 * 2 * kTileBytes;                // [2] per-visit vectors
    static constexpr int kYStage = kVec + 2 * kBlockVecBytes;            // [2] y of one chunk, bf16 tile
    static constexpr int kSStage = kYStage + 2 * kTileBytes;             // [2] state at a chunk start, bf16 [i][j] tile
    static constexpr int kGate = kSStage + 2 * kTileBytes;               // kFuse: [2] the gate's rows of one chunk
    static constexpr int kBytes = kGate + (kFuse ? 2 * kTileBytes : 0);
};
static_assert(BlockFwdLdsT<false>::kBytes <= 160 * 1024 && BlockFwdLdsT<true>::kBytes <= 160 * 1024, "LDS block of the block-form forward kernel");

struct BlockFwdArgs {
    int T, H, B;
    int bstep;               // batch rows between two pairs of a workgroup (B: one pair per workgroup)
    const bf16_t *r, *k, *v, *w, *u;
    const void *s0;          // initial state (B or n_state, H, 64, 64) [key][value] in Ts, or null
    const int64_t *map;      // batch row -> state row, or null
    bf16_t *y;
    void *sT;                // final state in Ts, or null
    float *ckpt;             // saved chunk states (bf16 [chunk][value][key] in the first half of each pair's slice), or null
    int *arrivals;           // with ckpt: per-head counters of the backward's fused gu sum, zeroed here
    // fused output stage (kFuse): out = (layer_norm over the head's 64 channels of y * gn_scale + gn_offset) * gate
    const bf16_t *gate;
    const float *gn_scale, *gn_offset;   // (H, 64)
    float gn_eps;
    bf16_t *out;
    float *stats;            // null, or (B, T, H, 2): mean and 1/sqrt(var + eps) per (token, head) for the backward
};

// sum over the 8 lanes that hold one 128-byte row (lanes 8k .. 8k+7), result in each of them
__device__ __forceinline__ float sum_row8(float x) {
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));   // row_half_mirror
    return x;
}

// ------------------------------------------------------------------------------------------
// Consumer wave q: value columns i = 16q + l16.
// State S[m]: rows j = block_row_channel(m, g) + rr, column i.
// ------------------------------------------------------------------------------------------
template <typename Ts, bool kSave, bool kFuse>
__device__ __forceinline__ void block_fwd_consumer(const BlockFwdArgs &a, unsigned char *smem, int pair0, int q, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int nchunk = (T + kBlockTokens - 1) / kBlockTokens;
    const int b0 = pair0 / H, h = pair0 - b0 * H;
    const int npw = (a.B - b0 + a.bstep - 1) / a.bstep;   // pairs of this workgroup: batch rows b0, b0 + bstep, ...
    const int nvisit = npw * nchunk;
    typedef BlockFwdLdsT<kFuse> BlockFwdLds;
    f32x4 S[4], Snext[4];
    // initial state of the workgroup's pair number `slot`, requested one visit before the pair begins
    auto request_state = [&](int slot) {
        const int b = b0 + slot * a.bstep;
        const int64_t row = a.map ? a.map[b] : (int64_t)b;
        const Ts *p = reinterpret_cast<const Ts *>(a.s0) + (row * H + h) * kN * kN + 16 * q + l16;
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) Snext[m][rr] = load1(p + (block_row_channel(m, g) + rr) * kN);
    };
    if (a.s0 != nullptr) request_state(0);
    if (kSave && b0 == 0 && q == 0 && lane == 0 && a.arrivals) a.arrivals[h] = 0;
    int c = 0, slot = 0;   // visit `it` is chunk c of pair number `slot`
    for (int it = 0; it < nvisit; ++it) {
        __syncthreads();
        if (c == 0) {
#pragma unroll
            for (int m = 0; m < 4; ++m) S[m] = a.s0 != nullptr ? Snext[m] : (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        if (a.s0 != nullptr && c == nchunk - 1 && slot + 1 < npw) request_state(slot + 1);
        const unsigned char *rt = smem + BlockFwdLds::kOp + (it & 1) * 2 * kTileBytes, *kt = rt + kTileBytes;
        const float *vec = reinterpret_cast<const float *>(smem + BlockFwdLds::kVec + (it & 1) * kBlockVecBytes);
        const float *ruk = vec + 4 * kN;
        const unsigned char *vt = smem + BlockFwdLds::kRawV + (it % (BlockFwdLds::kVAhead + 1)) * kTileBytes;
        if (kSave) {
            // the state at the chunk start, as the backward wants it: bf16, transposed ([i][j] rows of 128 bytes)
            unsigned char *ss = smem + BlockFwdLds::kSStage + (it & 1) * kTileBytes;
#pragma unroll
            for (int m = 0; m < 4; ++m)
                *reinterpret_cast<uint2 *>(ss + tile_off(16 * q + l16, block_row_channel(m, g))) =
                    make_uint2(pack_bf16x2(S[m][0], S[m][1]), pack_bf16x2(S[m][2], S[m][3]));
        }
        unsigned char *ys = smem + BlockFwdLds::kYStage + (it & 1) * kTileBytes;
        auto scale = [&](const float *gv) {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float4 gg = *reinterpret_cast<const float4 *>(&gv[block_row_channel(m, g)]);
                S[m][0] *= gg.x; S[m][1] *= gg.y; S[m][2] *= gg.z; S[m][3] *= gg.w;
            }
        };
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            scale(vec + 2 * blk * kN);   // g1 of the block
            {
                // y of this block's two 16-token row groups; products transposed (accumulator rows i = 4g + rr,
                // column t = l16: a lane holds four neighbouring channels of one token).  Every fragment is
                // fetched first, then the MFMAs run as independent chains.
                const bf16x8 sop0 = acc_as_operand(S[0], S[1]), sop1 = acc_as_operand(S[2], S[3]);
                const int r0 = 32 * blk + l16, r1 = r0 + 16;
                const bf16x8 rf0a = block_frag_ch(rt, r0, 0, g), rf0b = block_frag_ch(rt, r0, 1, g);
                const bf16x8 rf1a = block_frag_ch(rt, r1, 0, g), rf1b = block_frag_ch(rt, r1, 1, g);
                const bf16x8 kf0a = block_frag_ch(kt, r0, 0, g), kf0b = block_frag_ch(kt, r0, 1, g);
                const bf16x8 kf1a = block_frag_ch(kt, r1, 0, g), kf1b = block_frag_ch(kt, r1, 1, g);
                const s16x4 vf0 = tile_frag_tok(vt, 16 * q, 32 * blk, l16, g), vf1 = tile_frag_tok(vt, 16 * q, 32 * blk + 16, l16, g);
                const float ruk0 = ruk[r0], ruk1 = ruk[r1];
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                // A^T[s][t] = K~_s . R~_t (rows s = 4g + rr, column t = l16): blocks (0,0), (0,1), (1,1)
                f32x4 A00 = mfma32(kf0a, rf0a, zero), A01 = mfma32(kf0a, rf1a, zero), A11 = mfma32(kf1a, rf1a, zero);
                f32x4 Y0 = mfma32(sop0, rf0a, zero), Y1 = mfma32(sop0, rf1a, zero);
                A00 = mfma32(kf0b, rf0b, A00); A01 = mfma32(kf0b, rf1b, A01); A11 = mfma32(kf1b, rf1b, A11);
                Y0 = mfma32(sop1, rf0b, Y0); Y1 = mfma32(sop1, rf1b, Y1);
                settle(A00, A01, A11, Y0, Y1);
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int s_ = 4 * g + rr;
                    A00[rr] = (l16 > s_) ? A00[rr] : ((l16 == s_) ? ruk0 : 0.f);
                    A11[rr] = (l16 > s_) ? A11[rr] : ((l16 == s_) ? ruk1 : 0.f);
                }
                Y0 = mfma16(vf0, pack4(A00), Y0);
                Y1 = mfma16(vf0, pack4(A01), Y1);
                Y1 = mfma16(vf1, pack4(A11), Y1);
                settle(Y0, Y1);
                *reinterpret_cast<uint2 *>(ys + tile_off(r0, 16 * q + 4 * g)) = make_uint2(pack_bf16x2(Y0[0], Y0[1]), pack_bf16x2(Y0[2], Y0[3]));
                *reinterpret_cast<uint2 *>(ys + tile_off(r1, 16 * q + 4 * g)) = make_uint2(pack_bf16x2(Y1[0], Y1[1]), pack_bf16x2(Y1[2], Y1[3]));
            }
            // S <- g2 o (g1 o S + K~^T V) over the block's 32 tokens
            {
                s16x4 vf[2], kq[2][4];
#pragma unroll
                for (int pp = 0; pp < 2; ++pp) {
                    vf[pp] = tile_frag_tok(vt, 16 * q, 32 * blk + 16 * pp, l16, g);
#pragma unroll
                    for (int m = 0; m < 4; ++m) kq[pp][m] = block_frag_tok_rows(kt, m, 32 * blk + 16 * pp, l16, g);
                }
#pragma unroll
                for (int pp = 0; pp < 2; ++pp)
#pragma unroll
                    for (int m = 0; m < 4; ++m) S[m] = mfma16(kq[pp][m], vf[pp], S[m]);
            }
            settle(S[0], S[1], S[2], S[3]);
            scale(vec + (2 * blk + 1) * kN);   // g2 of the block
        }
        __builtin_amdgcn_sched_barrier(0);
        if (++c == nchunk) {
            if (a.sT != nullptr) {   // the pair's final state
                Ts *p = reinterpret_cast<Ts *>(a.sT) + ((int64_t)(b0 + slot * a.bstep) * H + h) * (kN * kN) + 16 * q + l16;
#pragma unroll
                for (int m = 0; m < 4; ++m)
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) store1(p + (block_row_channel(m, g) + rr) * kN, S[m][rr]);
            }
            c = 0;
            ++slot;
        }
    }
    __syncthreads();   // the producers write out the last chunk's staged rows behind this one
}

// ------------------------------------------------------------------------------------------
// Loading wave p (kRole = kBlockFwdLoads): tokens 16p..16p+15 of every chunk in, operands prepared.
// Storing wave p (kRole = kBlockFwdStores): the same rows of what the consumers staged, out.
// One function: both walk the same visits with the same cursors and lane mapping.
// ------------------------------------------------------------------------------------------
constexpr int kBlockFwdLoads = 1, kBlockFwdStores = 2;
template <bool kSave, bool kRagged, bool kFuse, int kRole>
__device__ __forceinline__ void block_fwd_producer(const BlockFwdArgs &a, unsigned char *smem, int *s_wild, int pair0, int p, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + kBlockTokens - 1) / kBlockTokens;
    const int b0 = pair0 / H, h = pair0 - b0 * H;
    const int npw = (a.B - b0 + a.bstep - 1) / a.bstep;
    const int nvisit = npw * nchunk;
    const uint32_t rowbytes = (uint32_t)C * 2u;
    const uint32_t lds0 = lds_address(smem);
    typedef BlockFwdLdsT<kFuse> BlockFwdLds;
    // first element of the workgroup's pair number `slot` in a (B,T,C) tensor
    auto pair_base = [&](int slot) { return (int64_t)(b0 + slot * a.bstep) * T * C + (int64_t)h * kN; };
    // this lane's part of an 8-row block: row (lane >> 3), 16-byte piece swizzled with the row
    const int lrow = lane >> 3;
    const uint32_t lpiece = (uint32_t)(((lane & 7) ^ lrow) << 4);
    // byte offset of this lane's piece of token row t of a pair (kRagged: rows past the end read the last row)
    auto row_offset = [&](int t) { return (uint32_t)(kRagged ? min(t, T - 1) : t) * rowbytes + lpiece; };
    // Every stream walks the flat sequence of visits (pair 0 chunk 0, 1, .., pair 1 chunk 0, ..) with a cursor
    // of its own: visit number `it`, its chunk `c`, and the pointers of its pair.
    struct Cursor {
        int it = 0, c = 0, slot = 0;
    };
    Cursor cv, cr, co, cp;   // v loads, r/k/w loads, stores of staged rows, operand preparation
    const bf16_t *vb = a.v + pair_base(0), *rb = a.r + pair_base(0), *kb_ = a.k + pair_base(0), *wb = a.w + pair_base(0);
    bf16_t *yb = (kFuse ? a.out : a.y) + pair_base(0);   // (kFuse: the rows that leave are those of `out`)
    bf16_t *y2b = kFuse && a.y ? a.y + pair_base(0) : nullptr;   // kFuse, training: y as well
    const bf16_t *gtb = kFuse ? a.gate + pair_base(0) : nullptr;
    // kFuse: scale and offset of the eight channels this lane holds of a row (the row's piece (lane & 7) ^ lrow),
    float gsc[8], gof[8];
    if (kFuse) {
        const float *sp = a.gn_scale + h * kN + (lpiece >> 1), *op_ = a.gn_offset + h * kN + (lpiece >> 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) { gsc[i] = sp[i]; gof[i] = op_[i]; }
    }
    char *ckb = kSave ? reinterpret_cast<char *>(a.ckpt + (int64_t)(b0 * H + h) * nchunk * (kN * kN)) : nullptr;
    // Vector-memory operations this wave has issued so far, and the count right after the r, k, w loads
    // of visit j went out: a wave's operations complete in program order, so "the loads of visit j have
    // landed" is "at most (issued - mark of j) operations are still in flight".
    int issued = 0, mark_even = 0, mark_odd = 0, mark_gate_even = 0, mark_gate_odd = 0;
    auto issue_v = [&]() {   // the next visit's v
        const uint32_t vv = lds0 + BlockFwdLds::kRawV + (cv.it % (BlockFwdLds::kVAhead + 1)) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
            load_rows8_to_lds(vb, row_offset(cv.c * kBlockTokens + 16 * p + 8 * blk + lrow), vv + 8 * blk * kTileRow);
        issued += 2;
        ++cv.it;
        if (++cv.c == nchunk) { cv.c = 0; ++cv.slot; vb = a.v + pair_base(cv.slot); }
    };
    auto issue_rkw = [&]() {   // the next visit's r, k, w
        const uint32_t raw = lds0 + BlockFwdLds::kRaw + (cr.it & 1) * 3 * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const uint32_t o = row_offset(cr.c * kBlockTokens + 16 * p + 8 * blk + lrow);
            load_rows8_to_lds(wb, o, raw + 2 * kTileBytes + 8 * blk * kTileRow);
            load_rows8_to_lds(rb, o, raw + 8 * blk * kTileRow);
            load_rows8_to_lds(kb_, o, raw + kTileBytes + 8 * blk * kTileRow);
        }
        issued += 6;
        if (cr.it & 1) mark_odd = issued; else mark_even = issued;
        ++cr.it;
        if (++cr.c == nchunk) {
            cr.c = 0; ++cr.slot;
            const int64_t nb = pair_base(cr.slot);
            rb = a.r + nb; kb_ = a.k + nb; wb = a.w + nb;
        }
    };
    // what the consumers staged during the next visit in line, as whole rows: y rows of this wave's tokens
    // and rows 16p..16p+15 of the chunk's state
    Cursor cg;   // kFuse: the gate's rows of a visit are requested when the visit begins and used one visit later
    auto issue_gate = [&]() {
        const uint32_t gg = lds0 + BlockFwdLds::kGate + (cg.it & 1) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
            load_rows8_to_lds(gtb, row_offset(cg.c * kBlockTokens + 16 * p + 8 * blk + lrow), gg + 8 * blk * kTileRow);
        issued += 2;
        if (cg.it & 1) mark_gate_odd = issued; else mark_gate_even = issued;
        ++cg.it;
        if (++cg.c == nchunk) { cg.c = 0; ++cg.slot; gtb = a.gate + pair_base(cg.slot); }
    };
    auto store_staged = [&]() {
        const unsigned char *ys = smem + BlockFwdLds::kYStage + (co.it & 1) * kTileBytes;
        const unsigned char *ss = smem + BlockFwdLds::kSStage + (co.it & 1) * kTileBytes;
        const unsigned char *gs = smem + BlockFwdLds::kGate + (co.it & 1) * kTileBytes;
        if (kFuse) wait_in_flight(issued - ((co.it & 1) ? mark_gate_odd : mark_gate_even));   // the visit's gate rows have landed
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const int row = 16 * p + 8 * blk + lrow, tok = co.c * kBlockTokens + row;
            const uint32_t o = (uint32_t)tok * rowbytes + lpiece;
            uint4 x = *reinterpret_cast<const uint4 *>(ys + row * kTileRow + (lane & 7) * 16);
            if (kFuse) {
                // the head's 64 channels of a token sit in eight neighbouring lanes: mean, variance (two passes, as
                // the unfused norm does it), scale, offset, gate
                if (y2b && (!kRagged || tok < T)) *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(y2b) + o) = x;
                float f[8], gt[8];
                const uint4 gx = *reinterpret_cast<const uint4 *>(gs + row * kTileRow + (lane & 7) * 16);
                unpack8(make_bf16x8(x.x, x.y, x.z, x.w), f);
                unpack8(make_bf16x8(gx.x, gx.y, gx.z, gx.w), gt);
                const float mean = sum_row8(((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]))) * (1.f / kN);
                float sq = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) { f[i] -= mean; sq = fmaf(f[i], f[i], sq); }
                const float rstd = __builtin_amdgcn_rsqf(sum_row8(sq) * (1.f / kN) + a.gn_eps);
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = fmaf(f[i] * rstd, gsc[i], gof[i]) * gt[i];
                x = make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
                if (a.stats && (lane & 7) == 0 && (!kRagged || tok < T))
                    *reinterpret_cast<float2 *>(a.stats + (((int64_t)(b0 + co.slot * a.bstep) * T + tok) * H + h) * 2) = make_float2(mean, rstd);
            }
            if (!kRagged || tok < T) *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(yb) + o) = x;
            if (kSave) {
                const uint4 s = *reinterpret_cast<const uint4 *>(ss + row * kTileRow + (lane & 7) * 16);
                *reinterpret_cast<uint4 *>(ckb + ((uint32_t)co.c * (uint32_t)(kN * kN * 2) + (uint32_t)(row * kTileRow) + lpiece)) = s;
            }
        }
        // (a store whose rows are all past the end is skipped: counting one that was not issued would let a later
        // wait return early, so only those that certainly went out are counted)
        issued += kSave ? 2 : 0;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const int rows_here = (!kRagged || co.c * kBlockTokens + 16 * p + 8 * blk < T) ? 1 : 0;
            issued += rows_here * (1 + (kFuse && y2b ? 1 : 0) + (kFuse && a.stats ? 1 : 0));
        }
        ++co.it;
        if (++co.c == nchunk) {
            co.c = 0; ++co.slot;
            yb = (kFuse ? a.out : a.y) + pair_base(co.slot);
            if (kFuse && y2b) y2b = a.y + pair_base(co.slot);
            if (kSave) ckb = reinterpret_cast<char *>(a.ckpt + (int64_t)((b0 + co.slot * a.bstep) * H + h) * nchunk * (kN * kN));
        }
    };
    float u4[4];
    load4(a.u + h * kN + 4 * l16, u4);   // (all pairs of a workgroup belong to one head)
    // the next visit in line (its r, k, w loads have been issued); `more`: the r, k, w loads of the next visit
    // not yet requested go out as soon as this one's raw rows are in registers (into the same LDS block)
    auto prepare = [&](bool more) {
        const int it = cp.it;
        const unsigned char *raw = smem + BlockFwdLds::kRaw + (it & 1) * 3 * kTileBytes;
        unsigned char *op = smem + BlockFwdLds::kOp + (it & 1) * 2 * kTileBytes;
        float *vec = reinterpret_cast<float *>(smem + BlockFwdLds::kVec + (it & 1) * kBlockVecBytes);
        wait_in_flight(issued - ((it & 1) ? mark_odd : mark_even));
        const bool ok = block_prepare<kRagged>(raw, raw + kTileBytes, raw + 2 * kTileBytes, vec, u4, p, l16, g, T - cp.c * kBlockTokens,
            [&]() {
                if (more) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    issue_rkw();
                }
            },
            [&](uint32_t o, const float (&xr)[4], const float (&xk)[4], const float (&)[4], const float (&)[4]) {
                *reinterpret_cast<uint2 *>(op + o) = make_uint2(pack_bf16x2(xr[0], xr[1]), pack_bf16x2(xr[2], xr[3]));
                *reinterpret_cast<uint2 *>(op + kTileBytes + o) = make_uint2(pack_bf16x2(xk[0], xk[1]), pack_bf16x2(xk[2], xk[3]));
            });
        if (!ok && lane == 0) s_wild[cp.slot] = 1;
        ++cp.it;
        if (++cp.c == nchunk) { cp.c = 0; ++cp.slot; }
    };
    // r, k, w of visit j are requested three visits ahead (two in the prologue), v kVAhead visits ahead
    constexpr int kVAhead = BlockFwdLds::kVAhead;
    if (kRole == kBlockFwdLoads) {
        issue_v();
        issue_rkw();
        if (nvisit > 1) { issue_v(); issue_rkw(); }
        if (kVAhead > 2 && nvisit > 2) issue_v();
        prepare(nvisit > 2);
    }
    for (int it = 0; it < nvisit; ++it) {
        __syncthreads();
        // free again: the raw v block of visit it-1; the staging tiles of visit it-1 are complete
        if (kRole == kBlockFwdLoads && it + kVAhead < nvisit) issue_v();
        if (kRole == kBlockFwdStores && kFuse) issue_gate();
        if (kRole == kBlockFwdStores && it > 0) store_staged();
        if (kRole == kBlockFwdLoads && it + 1 < nvisit) prepare(it + 3 < nvisit);
    }
    __syncthreads();
    if (kRole == kBlockFwdStores) store_staged();
    wait_loads<0>();
}

constexpr int kBlockFwdThreads = 12 * 64;

// the exact second pass leaves y in `out`; this turns one pair's rows into the fused output in place (a wave per
// token, lane = channel)
__device__ __forceinline__ void block_output_stage_in_place(const BlockFwdArgs &a, int b, int h) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = blockDim.x >> 6;
    const int64_t C = (int64_t)a.H * kN, first = (int64_t)b * a.T * C + (int64_t)h * kN + lane;
    const float gsc = a.gn_scale[h * kN + lane], gof = a.gn_offset[h * kN + lane];
    for (int t = wave; t < a.T; t += nwave) {
        const float y = load1(a.out + first + (int64_t)t * C);
        if (a.y) store1(a.y + first + (int64_t)t * C, y);
        float sum = y;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m);
        const float d = y - sum * (1.f / kN);
        float sq = d * d;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sq += __shfl_xor(sq, m);
        const float rstd = __builtin_amdgcn_rsqf(sq * (1.f / kN) + a.gn_eps);
        if (a.stats && lane == 0) *reinterpret_cast<float2 *>(a.stats + (((int64_t)b * a.T + t) * a.H + h) * 2) = make_float2(sum * (1.f / kN), rstd);
        store1(a.out + first + (int64_t)t * C, fmaf(d * rstd, gsc, gof) * load1(a.gate + first + (int64_t)t * C));
    }
}

template <typename Ts, bool kSave, bool kRagged, bool kFuse>
__global__ __launch_bounds__(kBlockFwdThreads) void block_fwd_kernel(BlockFwdArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild[kBlockMaxSlots];   // per pair of the workgroup: 16 tokens left the scaled operands' range
    static_assert(sizeof(ScanFwdLds) <= BlockFwdLdsT<kFuse>::kBytes, "the exact second pass reuses the LDS block");
    if (threadIdx.x < kBlockMaxSlots) s_wild[threadIdx.x] = 0;
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int pair0 = (int)blockIdx.x;
    if (wave < 4) block_fwd_producer<kSave, kRagged, kFuse, kBlockFwdLoads>(a, smem, s_wild, pair0, wave, lane);
    else if (wave < 8) block_fwd_consumer<Ts, kSave, kFuse>(a, smem, pair0, wave - 4, lane);
    else block_fwd_producer<kSave, kRagged, kFuse, kBlockFwdStores>(a, smem, s_wild, pair0, wave - 8, lane);
    // exact second pass for the pairs of which 16 tokens left the range the scaled operands can hold
    __threadfence_block();
    __syncthreads();
    const int b0 = pair0 / a.H, h = pair0 - b0 * a.H;
    const int npw = (a.B - b0 + a.bstep - 1) / a.bstep;
    for (int slot = 0; slot < npw; ++slot) {
        if (!s_wild[slot]) continue;   // (uniform over the workgroup)
        __syncthreads();
        scan_fwd_body<bf16_t, bf16_t, Ts>(*reinterpret_cast<ScanFwdLds *>(smem), b0 + slot * a.bstep, h, a.T, a.H, a.r, a.k, a.v, a.w, a.u,
                                          reinterpret_cast<const Ts *>(a.s0), a.map, kFuse ? a.out : a.y, reinterpret_cast<Ts *>(a.sT), false);
        if (kFuse) {
            __threadfence_block();
            __syncthreads();
            block_output_stage_in_place(a, b0 + slot * a.bstep, h);
        }
    }
}

// Workgroups of a launch: one per pair, or -- more pairs than compute units -- as many as there are compute
// units, rounded down to a multiple of H (so that a workgroup's pairs belong to one head); 0: the block form
// does not take the shape.
int64_t block_grid(int64_t B, int64_t H) {
    const int64_t pairs = B * H, cus = compute_units();
    if (pairs <= cus) return pairs;
    const int64_t grid = cus / H * H;
    // (heads that leave a tenth of the compute units idle, or more pairs per workgroup than its flags hold: tile form)
    if (grid * 10 < cus * 9 || (pairs + grid - 1) / grid > kBlockMaxSlots) return 0;
    return grid;
}

bool block_forward_applies(int64_t B, int64_t T, int64_t H) {
    const int64_t pairs = B * H, cus = compute_units();
    // (with fewer pairs than half the compute units the tile form shares a pair out over several workgroups)
    return 2 * pairs > cus && block_grid(B, H) > 0 && T * H * kN < (1LL << 31);
}

// gate != null: the fused output stage (out = (group norm of y) * gate; y and stats only where given)
static hipError_t block_forward_launch(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                                       const void *r, const void *k, const void *v, const void *w, const void *u,
                                       const void *s0, const int64_t *map, void *y, void *sT, void *saved_states, bool counters,
                                       const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps, void *out, float *stats)
{
    BlockFwdArgs a = {};
    a.T = (int)T; a.H = (int)H; a.B = (int)B;
    const int64_t grid = block_grid(B, H);
    a.bstep = B * H <= grid ? (int)B : (int)(grid / H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w; a.u = (const bf16_t *)u;
    a.s0 = s0; a.map = map; a.y = (bf16_t *)y; a.sT = sT; a.ckpt = (float *)saved_states;
    a.arrivals = saved_states && counters ? reinterpret_cast<int *>(reinterpret_cast<char *>(saved_states) + chunk_backward_workspace_bytes(B, T, H)) : nullptr;
    a.gate = (const bf16_t *)gate; a.gn_scale = gn_scale; a.gn_offset = gn_offset; a.gn_eps = gn_eps; a.out = (bf16_t *)out; a.stats = stats;
    auto launch = [&](auto ts_tag, auto save_tag, auto ragged_tag, auto fuse_tag) -> hipError_t {
        constexpr bool kFuse = decltype(fuse_tag)::value;
        constexpr auto kern = block_fwd_kernel<decltype(ts_tag), decltype(save_tag)::value, decltype(ragged_tag)::value, kFuse>;
        hipError_t e = allow_dynamic_lds<kern>(BlockFwdLdsT<kFuse>::kBytes);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kBlockFwdThreads), BlockFwdLdsT<kFuse>::kBytes, st, a);
        return hipGetLastError();
    };
    auto launch_ts = [&](auto ts_tag, auto save_tag, auto fuse_tag) -> hipError_t {
        return (T % kBlockTokens) != 0 ? launch(ts_tag, save_tag, std::true_type{}, fuse_tag) : launch(ts_tag, save_tag, std::false_type{}, fuse_tag);
    };
    const bool save = saved_states != nullptr;
    if (gate != nullptr) {
        // (the saving variant is the training one: zero initial state, no final state; its state type is immaterial)
        if (save) return launch_ts(float{}, std::true_type{}, std::true_type{});
        return state_dtype == kF32 ? launch_ts(float{}, std::false_type{}, std::true_type{}) : launch_ts(bf16_t{}, std::false_type{}, std::true_type{});
    }
    if (state_dtype == kF32) return save ? launch_ts(float{}, std::true_type{}, std::false_type{}) : launch_ts(float{}, std::false_type{}, std::false_type{});
    return save ? launch_ts(bf16_t{}, std::true_type{}, std::false_type{}) : launch_ts(bf16_t{}, std::false_type{}, std::false_type{});
}

hipError_t block_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states, bool counters)
{
    return block_forward_launch(st, state_dtype, B, T, H, r, k, v, w, u, s0, map, y, sT, saved_states, counters,
                                nullptr, nullptr, nullptr, 0.f, nullptr, nullptr);
}

hipError_t block_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s0, const int64_t *map, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                               void *out, void *y, float *stats, void *sT, void *saved_states)
{
    return block_forward_launch(st, state_dtype, B, T, H, r, k, v, w, u, s0, map, y, sT, saved_states, saved_states != nullptr,
                                gate, gn_scale, gn_offset, gn_eps, out, stats);
}

}  // namespace wkv6
