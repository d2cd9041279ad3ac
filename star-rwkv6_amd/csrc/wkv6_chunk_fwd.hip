// WKV6 in chunk-parallel form for gfx950: bf16 MFMA for the dense products, fp32 state.
//
// One workgroup (12 waves) per (batch, head) pair, or -- with more pairs than compute units -- one
// workgroup per compute unit that runs its pairs back to back through the same pipeline.  Time is
// cut into chunks of 64 tokens, each chunk into 4 tiles of 16 tokens.  The fp32 state S[j][i] lives in the MFMA accumulators of the
// "consumer" waves (wave q of a group owns value columns 16q..16q+15) and is advanced one tile at a time:
//
//   c_t = sum_{s<t} exp(w_s) inside the tile (so exp(-c_t) is the decay from the tile start to t)
//   R~[t][j] = r_t[j] exp(-c_t[j])            K~[t][j] = k_t[j] exp(+c_{t+1}[j])
//   g[j] = exp(-c_16[j])
//   A[t][s]  = R~_t . K~_s  (s < t),  A[t][t] = sum_j r_t[j] u[j] k_t[j]
//   Y        = R~ S + A V          (16x64x64 and 16x16x16 MFMA, K index j resp. s)
//   S       <- diag(g) (S + K~^T V)   (64x16x16 MFMA, K index s)
//
// Data path.  The raw r, k, w, v rows of a chunk go from global memory straight into LDS tiles
// (16-byte pieces, no registers), two chunks ahead of their use.  The four "producer" waves (one per
// tile, lane = channel) read r, k, w from there, compute R~, K~, g and the diagonal
// in fp32 for the NEXT chunk and write them back as bf16 tiles while the consumers run the MFMAs of
// the current one; the consumers (two groups of four waves that both carry the state but share out
// the per-tile output work) take V directly from its raw tile.  Every tile is stored once,
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
    static constexpr int kBytes0 = kOp + 2 * kOpBytes;
    // only WITHOUT the fused output stage: [2] K^ = K~ g, k decayed to the END of its tile (exponents <= 0)
    static constexpr int kKg = kBytes0;
    static constexpr int kBytes = kKg + 2 * kTileBytes;
    // only with the fused output stage (group norm and gate):
    static constexpr int kYStage = kBytes0;                             // [2 visit parities] y of one chunk, bf16
    static constexpr int kRawG = kYStage + 2 * kTileBytes;              // [4] raw gate tiles (visit & 3)
    static constexpr int kGnTab = kRawG + 4 * kTileBytes;               // [4][scale, offset][64] floats of the visit's head
    static constexpr int kBytesFused = kGnTab + 4 * 2 * kN * 4;
};

// With the fused output stage y does not go to global memory: the consumers leave each chunk in LDS
// as [token][64 channels] rows of 128 bytes, and a producer wave reads whole rows (lane = channel)
// one visit later.  The 32-byte slot of a consumer wave's 16 channels is XORed with bits 2..3 of the
// token, so that the four token rows one accumulator store touches fall into different banks.
__device__ __forceinline__ uint32_t ystage_off(int t, int ch) {
    return ((uint32_t)t << 7) + (((((uint32_t)ch >> 4) ^ ((uint32_t)t >> 2)) & 3u) << 5) + (((uint32_t)ch & 15u) << 1);
}

// Wave layout: 12 waves, four per role, one wave of each role per SIMD:
//   loader/producer (wave p <-> tile p) | consumer group 0 (y of tiles 0, 2) | consumer group 1 (tiles 1, 3)
constexpr int kFwdThreads = 12 * 64;

struct FwdArgs {
    int T, H;
    int nitems;      // B * H (batch, head) pairs; with kMulti a workgroup takes every gridDim.x-th of them
    int split;       // 1, 2 or 4 workgroups per pair, each with the consumer waves of 4 / split column slices
    int reverse;     // 1: the time axis is read back to front (row T-1-t in the place of row t); T a multiple of 64
    float *dsum;     // null, or [4 tiles][pairs][64]: per pair, log2(e) * sum of exp(w) over the tokens of tile p of every chunk
    const bf16_t *r, *k, *v, *w, *u;   // 16-bit elements: bf16, or fp16 with v a bf16 copy (see OutOf)
    const void *v_orig;                // v as the caller holds it (the exact per-timestep pass reads this one)
    const void *s0;
    const int64_t *map;
    bf16_t *y;
    void *sT;
    float *ckpt;
    int *arrivals;   // with ckpt: per-head counters the backward's fused gu sum starts from zero
    // fused output stage: out = (group_norm_head(y) * gn_scale + gn_offset) * gate, y itself is not written
    const bf16_t *gate;
    const float *gn_scale, *gn_offset;   // (H, 64)
    float gn_eps;
    bf16_t *out;
    // training with the fused output stage (then y above is written as well, for the norm's backward):
    float *stats;    // null, or (B, T, H, 2) fp32: mean and 1/sqrt(var + eps) of y over each head's channels
};

// ------------------------------------------------------------------------------------------
// Consumer group GRP of two: both groups carry the state through every tile (4 MFMAs and a
// scaling), group 0 produces y for tiles 0 and 2, group 1 for tiles 1 and 3.
// ------------------------------------------------------------------------------------------
template <typename Tin, typename Ts, bool kSave, bool kRagged, bool kMulti, bool kFuse, int GRP>
__device__ __forceinline__ void fwd_consumer(const FwdArgs &a, const unsigned char *smem, int bh0, int q, int lane)
{
    const int T = a.T, H = a.H;
    const int g = lane >> 4, l16 = lane & 15;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + CL - 1) / CL;
    const int stride = (int)gridDim.x;
    const int n_my = kMulti ? (a.nitems - bh0 + stride - 1) / stride : 1;
    const Ts *s0 = reinterpret_cast<const Ts *>(a.s0);
    // initial state of a (batch, head) pair as stored (converted when the pair starts)
    Ts Sraw[16];
    auto request_state = [&](int bh) {
        const int b = bh / H, h = bh - b * H;
        const int64_t row = a.map ? a.map[b] : (int64_t)b;
        const Ts *p = s0 + (row * H + h) * kN * kN + 16 * q + l16;
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) Sraw[4 * m + rr] = p[(16 * m + 4 * g + rr) * kN];
    };
    if (s0 != nullptr) request_state(bh0);
    int it = 0;   // chunk visits of this workgroup so far: picks the LDS buffers
    for (int n = 0, bh = bh0; n < n_my; ++n, bh += stride) {
        const int b = bh / H, h = bh - b * H;
        const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
        f32x4 S[4];
        if (s0 != nullptr) {
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) S[m][rr] = (float)Sraw[4 * m + rr];
        } else {
#pragma unroll
            for (int m = 0; m < 4; ++m) S[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        typedef typename OutOf<Tin>::type Tout;
        Tout *y_h = reinterpret_cast<Tout *>(a.y) + base;
        if (kSave && GRP == 0 && b == 0 && q == 0 && lane == 0 && a.arrivals) a.arrivals[h] = 0;
        for (int c = 0; c < nchunk; ++c, ++it) {
            __syncthreads();
            if (kSave && GRP == 0) {
                // The state at the chunk start goes to the workspace transposed, bf16 [chunk][i][j] in the
                // first half of this pair's slice: a lane's four rows j = 16m + 4g .. +3 of its column i are
                // eight contiguous bytes there, so a chunk takes four stores per lane.  They are issued behind
                // the barrier (the state registers do not change before the end of tile 0) and queue while
                // the other waves already work on the chunk.
                char *dst = reinterpret_cast<char *>(a.ckpt + (int64_t)bh * nchunk * (kN * kN)) + (int64_t)c * (kN * kN * 2) + (16 * q + l16) * (kN * 2) + 8 * g;
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    *reinterpret_cast<uint2 *>(dst + 32 * m) = make_uint2(pack_bf16x2(S[m][0], S[m][1]), pack_bf16x2(S[m][2], S[m][3]));
            }
            // the next pair's initial state is requested one chunk visit ahead of its use
            if (kMulti && s0 != nullptr && c == nchunk - 1 && n + 1 < n_my) request_state(bh + stride);
            // Tokens past the end were prepared as r = k = 0, decay 1: their tiles leave the state alone,
            // and their y rows are not stored.
            int op_off = FwdLds::kOp + (it & 1) * FwdLds::kOpBytes, v_off = FwdLds::kRawV + (it % 3) * kTileBytes;
            const int t0 = c * CL;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // (fresh_s: form the tile addresses per tile instead of holding them all across the chunk)
                const unsigned char *rt = smem + op_off + FwdLds::kOpRt, *kt = smem + op_off + FwdLds::kOpKt;
                const float *gv_ = reinterpret_cast<const float *>(smem + op_off + FwdLds::kOpG);
                const float *ruk = reinterpret_cast<const float *>(smem + op_off + FwdLds::kOpRuk);
                const unsigned char *vt = smem + v_off;
                const s16x4 vf = tile_frag_tok(vt, 16 * q, 16 * p, l16, g);
                const bool minep = (p & 1) == GRP && (kFuse || a.y != nullptr);   // (no y wanted: a pass that only builds the state)
                f32x4 U[4];
                bf16x8 sop0, sop1;
                if (minep) { sop0 = acc_as_operand(S[0], S[1]); sop1 = acc_as_operand(S[2], S[3]); }
                if (kFuse) {
                    // U = K~^T V in accumulators of its own, added to the state by VALU code at the end of the tile
#pragma unroll
                    for (int m = 0; m < 4; ++m) U[m] = mfma16(tile_frag_tok(kt, 16 * m, 16 * p, l16, g), vf, (f32x4){0.f, 0.f, 0.f, 0.f});
                } else {
                    // S <- diag(g) S + K^^T V: the new contributions' decay is folded into the operand, so the
                    // update is one scaling and an MFMA accumulation onto the state itself
                    const unsigned char *kgt = smem + FwdLds::kKg + (it & 1) * kTileBytes;
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const float4 gg = *reinterpret_cast<const float4 *>(&gv_[p * kN + 16 * m + 4 * g]);
                        S[m][0] *= gg.x; S[m][1] *= gg.y; S[m][2] *= gg.z; S[m][3] *= gg.w;
                    }
#pragma unroll
                    for (int m = 0; m < 4; ++m) S[m] = mfma16(tile_frag_tok(kgt, 16 * m, 16 * p, l16, g), vf, S[m]);
                }
                if (minep) {
                    const int row = 16 * p + l16;
                    const bf16x8 rf0 = tile_frag_ch(rt, row, 0, g), rf1 = tile_frag_ch(rt, row, 1, g);
                    const bf16x8 kf0 = tile_frag_ch(kt, row, 0, g), kf1 = tile_frag_ch(kt, row, 1, g);
                    const float rukv = ruk[row];
                    // A^T[s][t] = K~_s . R~_t  (accumulator rows s = 4g+r, column t = l16)
                    f32x4 AT = {0.f, 0.f, 0.f, 0.f};
                    AT = mfma32(kf0, rf0, AT);
                    AT = mfma32(kf1, rf1, AT);
                    // Y = R~ S
                    // Without the fused output stage the products are formed transposed (the operands change
                    // places): accumulator rows i = 4g + r, column t = l16, so that a lane holds four
                    // neighbouring channels of one token and writes them with one 8-byte store.
                    f32x4 Y = {0.f, 0.f, 0.f, 0.f};
                    if (kFuse) {
                        Y = mfma32(rf0, sop0, Y);
                        Y = mfma32(rf1, sop1, Y);
                    } else {
                        Y = mfma32(sop0, rf0, Y);
                        Y = mfma32(sop1, rf1, Y);
                    }
                    settle(AT);
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const int s = 4 * g + rr;
                        AT[rr] = (l16 > s) ? AT[rr] : ((l16 == s) ? rukv : 0.f);
                    }
                    // Y += A V : the masked A^T accumulator IS the operand holding A (token t = l16, k-slots s = 4g+r)
                    chain_gap(Y);
                    const s16x4 aop = make_s16x4(pack_bf16x2(AT[0], AT[1]), pack_bf16x2(AT[2], AT[3]));
                    Y = kFuse ? mfma16(aop, vf, Y) : mfma16(vf, aop, Y);
                    settle(Y);
                    if (kFuse) {
                        unsigned char *ys = const_cast<unsigned char *>(smem) + FwdLds::kYStage + (it & 1) * kTileBytes;
                        const uint32_t y01 = pack_bf16x2(Y[0], Y[1]), y23 = pack_bf16x2(Y[2], Y[3]);
                        const int tk = 16 * p + 4 * g, chn = 16 * q + l16;
                        *reinterpret_cast<uint16_t *>(ys + ystage_off(tk, chn)) = (uint16_t)y01;
                        *reinterpret_cast<uint16_t *>(ys + ystage_off(tk + 1, chn)) = (uint16_t)(y01 >> 16);
                        *reinterpret_cast<uint16_t *>(ys + ystage_off(tk + 2, chn)) = (uint16_t)y23;
                        *reinterpret_cast<uint16_t *>(ys + ystage_off(tk + 3, chn)) = (uint16_t)(y23 >> 16);
                    } else {
                        const int t = t0 + 16 * p + l16;   // channels 16q + 4g .. +3 of this token
                        if (!kRagged || t < T) store4(y_h + ((uint32_t)t * (uint32_t)C + (uint32_t)(16 * q + 4 * g)), Y[0], Y[1], Y[2], Y[3]);
                    }
                }
                if (kFuse) {
                    // S <- diag(g) (S + U)
                    settle(U[0], U[1], U[2], U[3]);
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        const float4 gg = *reinterpret_cast<const float4 *>(&gv_[p * kN + 16 * m + 4 * g]);
                        S[m][0] = (S[m][0] + U[m][0]) * gg.x; S[m][1] = (S[m][1] + U[m][1]) * gg.y;
                        S[m][2] = (S[m][2] + U[m][2]) * gg.z; S[m][3] = (S[m][3] + U[m][3]) * gg.w;
                    }
                } else {
                    settle(S[0], S[1], S[2], S[3]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (a.sT != nullptr && GRP == 0) {
            Ts *p = reinterpret_cast<Ts *>(a.sT) + (int64_t)bh * kN * kN + 16 * q + l16;
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) store1(p + (16 * m + 4 * g + rr) * kN, S[m][rr]);
        }
    }
    if (kFuse) __syncthreads();   // the producers finish the last visit's output behind this one
}

// ------------------------------------------------------------------------------------------
// Loader / producer, lane = channel: wave p <-> tile p of every chunk.
// ------------------------------------------------------------------------------------------
// kNoR: a pass that only builds states (no y wanted): r is neither loaded nor prepared
template <typename Tin, bool kSave, bool kRagged, bool kMulti, bool kFuse, bool kNoR>
__device__ __forceinline__ void fwd_producer(const FwdArgs &a, unsigned char *smem, int *s_wild, int bh0, int part, int pw, int lane)
{
    constexpr int NT = 16;   // tokens per wave and chunk
    const int T = a.T, H = a.H;
    const int p = pw;
    const int ch = lane;
    const int64_t C = (int64_t)H * kN;
    const int nchunk = (T + CL - 1) / CL;
    const int stride = (int)gridDim.x;
    const int n_my = kMulti ? (a.nitems - bh0 + stride - 1) / stride : 1;
    const int nvisit = n_my * nchunk;   // chunk visits of this workgroup, pair after pair
    const uint32_t rowbytes = (uint32_t)C * 2u;
    const uint32_t lds0 = lds_address(smem);
    // this lane's part of an 8-row block load: row (lane >> 3), 16-byte piece swizzled with the row
    const int lrow = lane >> 3;
    const uint32_t lpiece = (uint32_t)(((lane & 7) ^ lrow) << 4);
    // The load stream and the preparation stream each walk the visits in order; `ld_*` / `pp_*` are
    // the (pair, chunk) the next load / preparation belongs to.
    int ld_c = 0, ld_bh = bh0, ld_h = 0;
    const bf16_t *rb, *kb_, *vb, *wb, *gb = nullptr;   // uniform: this pair's first row (gb: gate, fused output stage)
    auto point_loads = [&]() {
        const int b = ld_bh / H, h = ld_bh - b * H;
        ld_h = h;
        const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
        rb = a.r + base; kb_ = a.k + base; vb = a.v + base; wb = a.w + base;
        if (kFuse) gb = a.gate + base;
    };
    point_loads();
    // Rows past the end of the sequence are fetched from row T-1 (valid memory); the operand
    // preparation turns them into r = k = 0, w = -inf (decay 1), and the v rows only ever meet zero
    // operands.  Each wave loads what it reads itself, so its own vmcnt covers its inputs; v is
    // picked up by the consumers a barrier later.
    constexpr int kLoads = 8 + (kFuse ? 2 : 0) - (kNoR ? 2 : 0);   // per chunk and wave
    constexpr int kLoads0 = kLoads + (kFuse ? 2 : 0);                  // wave 0 also brings the norm's scale and offset
    auto issue_loads = [&](int it) {   // visit `it` = the load stream's current (pair, chunk)
        const int tb = ld_c * CL + 16 * p;
        const uint32_t rkw = lds0 + FwdLds::kRawRKW + (it & 1) * 3 * kTileBytes + 16 * p * kTileRow;
        const uint32_t vv = lds0 + FwdLds::kRawV + (it % 3) * kTileBytes + 16 * p * kTileRow;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const int t = tb + 8 * blk + lrow;
            const uint32_t o = (uint32_t)(kRagged ? min(t, T - 1) : a.reverse ? T - 1 - t : t) * rowbytes + lpiece;
            load_rows8_to_lds(wb, o, rkw + 2 * kTileBytes + 8 * blk * kTileRow);
            if (!kNoR) load_rows8_to_lds(rb, o, rkw + 8 * blk * kTileRow);
            load_rows8_to_lds(kb_, o, rkw + kTileBytes + 8 * blk * kTileRow);
            load_rows8_to_lds(vb, o, vv + 8 * blk * kTileRow);
            if (kFuse) load_rows8_to_lds(gb, o, lds0 + FwdLds::kRawG + (it & 3) * kTileBytes + (16 * p + 8 * blk) * kTileRow);
        }
        if (kFuse && pw == 0 && lane < 16) {
            // scale and offset of this visit's head (64 floats each), read by all four waves' output stage
            const uint32_t tab = lds0 + FwdLds::kGnTab + (it & 3) * (2 * kN * 4);
            load_rows8_to_lds(a.gn_scale + ld_h * kN, (uint32_t)lane * 16u, tab);
            load_rows8_to_lds(a.gn_offset + ld_h * kN, (uint32_t)lane * 16u, tab + kN * 4);
        }
        if (++ld_c == nchunk && kMulti) { ld_c = 0; ld_bh += stride; if (ld_bh < a.nitems) point_loads(); }
    };
    // waits until at most `stores` + this wave's loads of one visit are in flight
    auto wait_visit_loads = [&](bool next_in_flight, bool stores_behind) {
        if (next_in_flight) {
            if (stores_behind) { if (pw == 0) wait_loads<kLoads0 + 16>(); else wait_loads<kLoads + 16>(); }
            else { if (pw == 0) wait_loads<kLoads0>(); else wait_loads<kLoads>(); }
        } else {
            if (stores_behind) wait_loads<16>(); else wait_loads<0>();
        }
    };
    // per-lane byte offsets of channel `ch` inside a tile row, for the 8 swizzle phases
    uint32_t choff[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) choff[s] = (uint32_t)((((ch >> 3) ^ s) << 4) + ((ch & 7) << 1)) + (uint32_t)(16 * p * kTileRow);
    // Fused output stage for the chunk the consumers staged during the previous visit; wave p takes
    // tile p, lane = channel:  out = ((y - mean) * rstd * gn_scale + gn_offset) * gate, mean and
    // variance over the head's 64 channels of a token (two passes, like a layer norm).
    int fl_c = 0, fl_bh = bh0;
    bf16_t *ob = nullptr, *yb = nullptr;
    float *sb = nullptr;
    constexpr bool train = kFuse && kSave;   // training: y and the norm's statistics are written too
    auto point_output = [&]() {
        const int b = fl_bh / H, h = fl_bh - b * H;
        ob = a.out + (int64_t)b * T * C + (int64_t)h * kN;
        if (train) { yb = a.y + (int64_t)b * T * C + (int64_t)h * kN; sb = a.stats + ((int64_t)b * T * H + h) * 2; }
    };
    if (kFuse) point_output();
    auto output_stage = [&](int it) {   // visit `it` = the output stream's current (pair, chunk)
        const unsigned char *ys = smem + FwdLds::kYStage + (it & 1) * kTileBytes;
        const unsigned char *gt = smem + FwdLds::kRawG + (it & 3) * kTileBytes;
        const float *tab = reinterpret_cast<const float *>(smem + FwdLds::kGnTab + (it & 3) * (2 * kN * 4));
        const float gsc = tab[ch], gof = tab[kN + ch];
        float yv[16], dv[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t bits = *reinterpret_cast<const uint16_t *>(ys + ystage_off(16 * p + e, ch));
            yv[e] = bf16_bits_to_float(bits);
            const int t = fl_c * CL + 16 * p + e;
            if (train && (!kRagged || t < T)) *reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(yb) + ((uint32_t)t * rowbytes + 2u * (uint32_t)ch)) = (uint16_t)bits;
        }
        // lane l of the reduction holds the total of token (l >> 2) & 15
        const float mu_own = transpose_reduce16(yv, lane) * (1.f / kN);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float mu = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mu_own), 4 * e));
            yv[e] -= mu;
            dv[e] = yv[e] * yv[e];
        }
        const float rstd_own = __builtin_amdgcn_rsqf(transpose_reduce16(dv, lane) * (1.f / kN) + a.gn_eps);
        if (train && (lane & 3) == 0) {
            const int t = fl_c * CL + 16 * p + ((lane >> 2) & 15);
            if (!kRagged || t < T) *reinterpret_cast<float2 *>(sb + (int64_t)t * H * 2) = make_float2(mu_own, rstd_own);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float rstd = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(rstd_own), 4 * e));
            const float gate = bf16_bits_to_float(*reinterpret_cast<const uint16_t *>(gt + choff[e & 7] + e * kTileRow));
            const int t = fl_c * CL + 16 * p + e;
            const float o = fmaf(yv[e] * rstd, gsc, gof) * gate;
            if (!kRagged || t < T) st16(ob, (uint32_t)t * rowbytes + 2u * (uint32_t)ch, o);
        }
        if (++fl_c == nchunk && kMulti) { fl_c = 0; fl_bh += stride; if (fl_bh < a.nitems) point_output(); }
    };
    int pp_c = 0, pp_n = 0, pp_h = bh0 % H;
    float uc = load1(reinterpret_cast<const Tin *>(a.u) + pp_h * kN + ch);
    float dacc = 0.f;   // base-2 decay exponent summed over this wave's tiles of the current pair
    const float kLog2Log2e = 0.5287663729448977f;   // log2(log2(e)): exp(w) log2(e) = 2^(w log2(e) + this)
    auto prepare = [&](int it) {   // visit `it` = the preparation stream's current (pair, chunk)
        const unsigned char *raw = smem + FwdLds::kRawRKW + (it & 1) * 3 * kTileBytes;
        unsigned char *op = smem + FwdLds::kOp + (it & 1) * FwdLds::kOpBytes;
        const int tb = pp_c * CL + 16 * p;
        // exponents are kept in base 2 (one v_exp_f32 each, no extra scaling multiply)
        float cs2 = 0.f, pa = 1.f;
        float fr[NT], fk[NT], fw[NT];
#pragma unroll
        for (int e = 0; e < NT; ++e) {
            const uint32_t o = choff[e & 7] + e * kTileRow;
            uint32_t ra = kNoR ? 0u : *reinterpret_cast<const uint16_t *>(raw + o);
            uint32_t rk = *reinterpret_cast<const uint16_t *>(raw + kTileBytes + o);
            uint32_t rw = *reinterpret_cast<const uint16_t *>(raw + 2 * kTileBytes + o);
            if (kRagged && tb + e >= T) { ra = 0u; rk = 0u; rw = neg_inf_bits<Tin>(); }
            fr[e] = in_bits_to_float<Tin>(ra); fk[e] = in_bits_to_float<Tin>(rk); fw[e] = in_bits_to_float<Tin>(rw);
        }
        float xr[NT], xk[NT], pr[NT];
#pragma unroll
        for (int e = 0; e < NT; ++e) {
            const float ew2 = exp2_fast(fmaf(fw[e], kLog2e, kLog2Log2e));   // exp(w) * log2(e)
            xr[e] = fr[e] * pa;               // r exp(-c_t)
            cs2 += ew2;
            xk[e] = fk[e] * exp2_fast(cs2);   // k exp(+c_{t+1})
            pa *= exp2_fast(-ew2);
            pr[e] = fr[e] * uc * fk[e];
        }
#pragma unroll
        for (int e = 0; e < NT; e += 2) {
            const uint32_t pr2 = pack_bf16x2(xr[e], xr[e + 1]), pk2 = pack_bf16x2(xk[e], xk[e + 1]);
            const uint32_t o0 = choff[e & 7] + e * kTileRow, o1 = choff[(e + 1) & 7] + (e + 1) * kTileRow;
            if (!kNoR) {
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpRt + o0) = (uint16_t)pr2;
                *reinterpret_cast<uint16_t *>(op + FwdLds::kOpRt + o1) = (uint16_t)(pr2 >> 16);
            }
            *reinterpret_cast<uint16_t *>(op + FwdLds::kOpKt + o0) = (uint16_t)pk2;
            *reinterpret_cast<uint16_t *>(op + FwdLds::kOpKt + o1) = (uint16_t)(pk2 >> 16);
        }
        if (!kFuse) {
            // K^ = K~ g = k exp(-(c_16 - c_{t+1})): the state update's operand
            unsigned char *kg = smem + FwdLds::kKg + (it & 1) * kTileBytes;
#pragma unroll
            for (int e = 0; e < NT; e += 2) {
                const uint32_t pg2 = pack_bf16x2(xk[e] * pa, xk[e + 1] * pa);
                const uint32_t o0 = choff[e & 7] + e * kTileRow, o1 = choff[(e + 1) & 7] + (e + 1) * kTileRow;
                *reinterpret_cast<uint16_t *>(kg + o0) = (uint16_t)pg2;
                *reinterpret_cast<uint16_t *>(kg + o1) = (uint16_t)(pg2 >> 16);
            }
        }
        // the whole tile's decay: g, and the range check of exp(+c)
        if (__builtin_amdgcn_ballot_w64(!(cs2 <= kWildLimit * kLog2e)) != 0ull) {
            if (lane == 0) s_wild[pp_n] = 1;
        }
        dacc += cs2;
        reinterpret_cast<float *>(op + FwdLds::kOpG)[p * kN + ch] = pa;
        if (!kNoR) {
            const float tot = transpose_reduce16(pr, lane);
            if ((lane & 3) == 0) reinterpret_cast<float *>(op + FwdLds::kOpRuk)[16 * p + ((lane >> 2) & 15)] = tot;
        }
        if (pp_c + 1 == nchunk && a.dsum != nullptr && part == 0) {   // the pair's total decay, this wave's tiles
            a.dsum[((int64_t)p * a.nitems + (bh0 + pp_n * stride)) * kN + ch] = dacc;
            dacc = 0.f;
        }
        if (++pp_c == nchunk && kMulti) {   // the next preparation opens the next pair: its head's u
            pp_c = 0; ++pp_n;
            if (pp_n < n_my) {
                pp_h = (bh0 + pp_n * stride) % H;
                uc = load1(reinterpret_cast<const Tin *>(a.u) + pp_h * kN + ch);
            }
        }
    };
    // visit `it` is loaded during visit it-2 (or the prologue), prepared during visit it-1
    issue_loads(0);
    if (nvisit > 1) issue_loads(1);
    wait_visit_loads(nvisit > 1, false);
    prepare(0);
    for (int it = 0; it < nvisit; ++it) {
        __syncthreads();
        // the raw r, k, w block of visit `it` (read by this wave's prepare(it) before the barrier) and the
        // raw v block of visit it-1 (read by the consumers before the barrier) are free again.
        // The output stage's 16 stores go out behind the loads and are not waited for: a wave's
        // memory operations complete in program order, and the loads waited for below are older
        // than both.  (With a ragged end the number of store instructions issued is not fixed;
        // they go first then and are waited for with the loads.)
        const bool outputs = kFuse && it > 0;
        const bool stores_first = kRagged || train;   // (training writes y and the statistics too: not the fixed 16 stores)
        if (outputs && stores_first) output_stage(it - 1);
        if (it + 2 < nvisit) issue_loads(it + 2);
        if (outputs && !stores_first) output_stage(it - 1);
        if (it + 1 < nvisit) {
            wait_visit_loads(it + 2 < nvisit, outputs && !stores_first);
            prepare(it + 1);
        }
    }
    if (kFuse) {
        __syncthreads();
        output_stage(nvisit - 1);
    }
    wait_loads<0>();
}

// kMulti: more (batch, head) pairs than workgroups -- each workgroup takes every gridDim.x-th pair and
// runs them back to back through one pipeline, so the loads of a pair's first chunks overlap the
// previous pair's last ones (a workgroup fills the CU's LDS, so nothing else would hide them).
constexpr int kMaxPairsPerWorkgroup = 32;
// The exact second pass leaves y in `out`; this turns one pair's rows into the fused output in place
// (a wave per token, lane = channel).
__device__ __forceinline__ void output_stage_in_place(const FwdArgs &a, int bh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = blockDim.x >> 6;
    const int b = bh / a.H, h = bh - b * a.H;
    const int64_t C = (int64_t)a.H * kN;
    bf16_t *rowp = a.out + (int64_t)b * a.T * C + (int64_t)h * kN + lane;
    const bf16_t *gp = a.gate + (int64_t)b * a.T * C + (int64_t)h * kN + lane;
    const float gsc = a.gn_scale[h * kN + lane], gof = a.gn_offset[h * kN + lane];
    for (int t = wave; t < a.T; t += nwave) {
        const float y = load1(rowp + (int64_t)t * C);
        if (a.y) store1(a.y + (int64_t)b * a.T * C + (int64_t)h * kN + lane + (int64_t)t * C, y);
        float sum = y;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m);
        const float d = y - sum * (1.f / kN);
        float sq = d * d;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sq += __shfl_xor(sq, m);
        const float rstd = __builtin_amdgcn_rsqf(sq * (1.f / kN) + a.gn_eps);
        if (a.stats && lane == 0) *reinterpret_cast<float2 *>(a.stats + (((int64_t)b * a.T + t) * a.H + h) * 2) = make_float2(sum * (1.f / kN), rstd);
        store1(rowp + (int64_t)t * C, fmaf(d * rstd, gsc, gof) * load1(gp + (int64_t)t * C));
    }
}

template <typename Tin, typename Ts, bool kSave, bool kRagged, bool kMulti, bool kFuse, bool kNoR = false>
__global__ __launch_bounds__(kFwdThreads) void chunk_fwd_kernel(FwdArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_wild[kMaxPairsPerWorkgroup];
    static_assert(sizeof(ScanFwdLds) <= FwdLds::kBytes, "the exact second pass reuses the LDS block");
    if (threadIdx.x < kMaxPairsPerWorkgroup) s_wild[threadIdx.x] = 0;
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // With fewer pairs than compute units a pair is shared by `split` workgroups: the value columns of
    // the state are independent of each other, so each workgroup carries the consumer waves of its
    // 4 / split column slices (and repeats the operand preparation, which does not depend on them).
    const int split = kMulti || kFuse ? 1 : a.split;
    const int bh0 = (int)blockIdx.x / split, part = (int)blockIdx.x - bh0 * split;
    const int nq = 4 / split;   // consumer waves per group
    if (wave < 4) {
        fwd_producer<Tin, kSave, kRagged, kMulti, kFuse, kNoR>(a, smem, s_wild, bh0, part, wave, lane);
    } else {
        const int cw = wave - 4, grp = cw / nq, q = part * nq + (cw - grp * nq);
        if (grp == 0) fwd_consumer<Tin, Ts, kSave, kRagged, kMulti, kFuse, 0>(a, smem, bh0, q, lane);
        else fwd_consumer<Tin, Ts, kSave, kRagged, kMulti, kFuse, 1>(a, smem, bh0, q, lane);
    }
    // exact second pass for every pair of this workgroup that had a tile leave the representable range
    // (workgroups sharing a pair all see the same flags and all redo the whole pair: the same values)
    __threadfence_block();   // workgroup scope is enough (and a device-scope fence would write back the L2)
    __syncthreads();
    const int stride = (int)gridDim.x;
    const int n_my = kMulti ? (a.nitems - bh0 + stride - 1) / stride : 1;
    for (int n = 0; n < n_my; ++n) {
        if (!s_wild[n]) continue;   // uniform over the workgroup
        const int bh = bh0 + n * stride;
        __syncthreads();
        typedef typename OutOf<Tin>::type Tout;
        auto in = [](const void *p) { return reinterpret_cast<const Tin *>(p); };
        scan_fwd_body<Tin, Tout, Ts>(*reinterpret_cast<ScanFwdLds *>(smem), bh / a.H, bh % a.H, a.T, a.H, in(a.r), in(a.k), in(a.v_orig), in(a.w), in(a.u),
                                     reinterpret_cast<const Ts *>(a.s0), a.map, reinterpret_cast<Tout *>(kFuse ? a.out : a.y), reinterpret_cast<Ts *>(a.sT), a.reverse != 0);
        if (kFuse) {
            __threadfence_block();
            __syncthreads();
            output_stage_in_place(a, bh);
        }
    }
}

// compute units of the current device (an immutable device property, looked up once per device)
int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

template <typename Tin, typename Ts, bool kSave, bool kRagged, bool kMulti, bool kFuse, bool kNoR = false>
static hipError_t launch_fwd(hipStream_t st, const FwdArgs &a, unsigned grid) {
    constexpr auto kern = chunk_fwd_kernel<Tin, Ts, kSave, kRagged, kMulti, kFuse, kNoR>;
    const size_t lds = kFuse ? FwdLds::kBytesFused : FwdLds::kBytes;
    hipError_t e = allow_dynamic_lds<kern>((int)lds);
    if (e != hipSuccess) return e;
    const int split = kMulti || kFuse ? 1 : a.split;
    hipLaunchKernelGGL(kern, dim3(grid * split), dim3((4 + 8 / split) * 64), lds, st, a);
    return hipGetLastError();
}
template <typename Tin, typename Ts, bool kSave, bool kRagged, bool kFuse>
static hipError_t launch_fwd(hipStream_t st, const FwdArgs &a, bool multi, unsigned grid) {
    // no y wanted and fp32 states (the state-only passes of the backward and of the time segments):
    // the variant that leaves r alone
    if constexpr (!kFuse && std::is_same<Ts, float>::value && std::is_same<Tin, bf16_t>::value) {
        if (a.y == nullptr)
            return multi ? launch_fwd<Tin, Ts, kSave, kRagged, true, kFuse, true>(st, a, grid)
                         : launch_fwd<Tin, Ts, kSave, kRagged, false, kFuse, true>(st, a, grid);
    }
    return multi ? launch_fwd<Tin, Ts, kSave, kRagged, true, kFuse>(st, a, grid) : launch_fwd<Tin, Ts, kSave, kRagged, false, kFuse>(st, a, grid);
}
template <typename Ts>
static hipError_t launch_fwd(hipStream_t st, const FwdArgs &a, bool save, bool ragged, bool multi, unsigned grid) {
    if (save) return ragged ? launch_fwd<bf16_t, Ts, true, true, false>(st, a, multi, grid) : launch_fwd<bf16_t, Ts, true, false, false>(st, a, multi, grid);
    return ragged ? launch_fwd<bf16_t, Ts, false, true, false>(st, a, multi, grid) : launch_fwd<bf16_t, Ts, false, false, false>(st, a, multi, grid);
}
template <typename Ts>
static hipError_t launch_fwd_fused(hipStream_t st, const FwdArgs &a, bool ragged, bool multi, unsigned grid) {
    return ragged ? launch_fwd<bf16_t, Ts, false, true, true>(st, a, multi, grid) : launch_fwd<bf16_t, Ts, false, false, true>(st, a, multi, grid);
}

// One workgroup per pair while they all fit on the chip at once; beyond that one workgroup per
// compute unit (more only if a workgroup would otherwise get more pairs than it keeps flags for).
static unsigned forward_grid(int64_t pairs, bool *multi, int *split) {
    const int64_t cus = compute_units();
    *multi = pairs > cus;
    *split = pairs * 4 <= cus ? 4 : pairs * 2 <= cus ? 2 : 1;
    return (unsigned)(!*multi ? pairs : (pairs + cus * kMaxPairsPerWorkgroup - 1) / (cus * kMaxPairsPerWorkgroup) * cus);
}

hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states, float *dsum, bool reverse,
                         bool counters)
{
    if (y != nullptr && dsum == nullptr && !reverse && block_forward_applies(B, T, H))
        return block_forward(st, state_dtype, B, T, H, r, k, v, w, u, s0, map, y, sT, saved_states, counters);
    FwdArgs a = {};
    a.dsum = dsum;
    a.reverse = reverse && (T % CL) == 0;
    a.T = (int)T; a.H = (int)H; a.nitems = (int)(B * H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w; a.u = (const bf16_t *)u;
    a.v_orig = v;
    a.s0 = s0; a.map = map; a.y = (bf16_t *)y; a.sT = sT; a.ckpt = (float *)saved_states;
    a.arrivals = saved_states && counters ? reinterpret_cast<int *>(reinterpret_cast<char *>(saved_states) + chunk_backward_workspace_bytes(B, T, H)) : nullptr;
    bool multi;
    const unsigned grid = forward_grid(B * H, &multi, &a.split);
    const bool save = saved_states != nullptr, ragged = (T % CL) != 0;
    return state_dtype == kF32 ? launch_fwd<float>(st, a, save, ragged, multi, grid)
                               : launch_fwd<bf16_t>(st, a, save, ragged, multi, grid);
}

// bf16 copy of an fp16 or fp32 tensor (n a multiple of 8 elements, 16-byte aligned): what the MFMAs take as v and gy
template <typename Tsrc>
__global__ __launch_bounds__(256) void to_bf16_kernel(const Tsrc *__restrict__ src, bf16_t *__restrict__ dst, int64_t n8)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        Raw8<Tsrc> x;
        x.load(src + 8 * i);
        float f[8];
        x.to_float(f);
        *reinterpret_cast<uint4 *>(dst + 8 * i) = make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
    }
}
hipError_t convert_to_bf16(hipStream_t st, int src_dtype, const void *src, void *dst, int64_t n)
{
    const int64_t n8 = n / 8;
    const unsigned grid = (unsigned)((n8 + 255) / 256 < 16384 ? (n8 + 255) / 256 : 16384);
    if (src_dtype == kF16) hipLaunchKernelGGL(to_bf16_kernel<f16_t>, dim3(grid), dim3(256), 0, st, (const f16_t *)src, (bf16_t *)dst, n8);
    else hipLaunchKernelGGL(to_bf16_kernel<float>, dim3(grid), dim3(256), 0, st, (const float *)src, (bf16_t *)dst, n8);
    return hipGetLastError();
}

// The saving forward of the training pair for fp16 tensors (y fp32, zero initial state): r, k, w are
// read as fp16 and unpacked exactly, v_bf16 is the bf16 copy of v the MFMAs take.
hipError_t chunk_forward_save_f16(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                  const void *r, const void *k, const void *v, const void *v_bf16, const void *w, const void *u,
                                  void *y, void *saved_states)
{
    FwdArgs a = {};
    a.T = (int)T; a.H = (int)H; a.nitems = (int)(B * H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v_bf16; a.w = (const bf16_t *)w; a.u = (const bf16_t *)u;
    a.v_orig = v;
    a.y = (bf16_t *)y; a.ckpt = (float *)saved_states;
    a.arrivals = reinterpret_cast<int *>(reinterpret_cast<char *>(saved_states) + chunk_backward_workspace_bytes(B, T, H));
    bool multi;
    const unsigned grid = forward_grid(B * H, &multi, &a.split);
    return (T % CL) != 0 ? launch_fwd<f16_t, float, true, true, false>(st, a, multi, grid)
                         : launch_fwd<f16_t, float, true, false, false>(st, a, multi, grid);
}

hipError_t chunk_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s0, const int64_t *map, const void *gate, const float *gn_scale,
                               const float *gn_offset, float gn_eps, void *out, void *sT)
{
    if (block_forward_applies(B, T, H))
        return block_forward_fused(st, state_dtype, B, T, H, r, k, v, w, u, s0, map, gate, gn_scale, gn_offset, gn_eps, out, nullptr, nullptr, sT, nullptr);
    FwdArgs a = {};
    a.T = (int)T; a.H = (int)H; a.nitems = (int)(B * H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w; a.u = (const bf16_t *)u;
    a.s0 = s0; a.map = map; a.sT = sT;
    a.v_orig = v;
    a.gate = (const bf16_t *)gate; a.gn_scale = gn_scale; a.gn_offset = gn_offset; a.gn_eps = gn_eps; a.out = (bf16_t *)out;
    bool multi;
    const unsigned grid = forward_grid(B * H, &multi, &a.split);
    a.split = 1;   // the output stage needs a chunk's whole rows in one workgroup
    const bool ragged = (T % CL) != 0;
    return state_dtype == kF32 ? launch_fwd_fused<float>(st, a, ragged, multi, grid)
                               : launch_fwd_fused<bf16_t>(st, a, ragged, multi, grid);
}

// Training with the fused output stage: out = (group_norm_head(y) * gn_scale + gn_offset) * gate, and for
// the backward y itself (bf16), the norm's statistics and the chunk states.  s0: null (zero initial state: what
// the caller sees), or one fp32 state per pair (a segment's incoming state).
static hipError_t fused_save_from(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                  const void *r, const void *k, const void *v, const void *w, const void *u, const float *s0,
                                  const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                                  void *out, void *y, float *stats, void *saved_states)
{
    if (block_forward_applies(B, T, H))
        return block_forward_fused(st, kF32, B, T, H, r, k, v, w, u, s0, nullptr, gate, gn_scale, gn_offset, gn_eps, out, y, stats, nullptr, saved_states);
    FwdArgs a = {};
    a.s0 = s0;
    a.T = (int)T; a.H = (int)H; a.nitems = (int)(B * H);
    a.r = (const bf16_t *)r; a.k = (const bf16_t *)k; a.v = (const bf16_t *)v; a.w = (const bf16_t *)w; a.u = (const bf16_t *)u;
    a.v_orig = v;
    a.gate = (const bf16_t *)gate; a.gn_scale = gn_scale; a.gn_offset = gn_offset; a.gn_eps = gn_eps; a.out = (bf16_t *)out;
    a.y = (bf16_t *)y; a.stats = stats; a.ckpt = (float *)saved_states;
    a.arrivals = reinterpret_cast<int *>(reinterpret_cast<char *>(saved_states) + chunk_backward_workspace_bytes(B, T, H));
    bool multi;
    const unsigned grid = forward_grid(B * H, &multi, &a.split);
    a.split = 1;
    return (T % CL) != 0 ? launch_fwd<bf16_t, float, true, true, true>(st, a, multi, grid)
                         : launch_fwd<bf16_t, float, true, false, true>(st, a, multi, grid);
}
hipError_t chunk_forward_fused_save(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                    const void *r, const void *k, const void *v, const void *w, const void *u,
                                    const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                                    void *out, void *y, float *stats, void *saved_states)
{
    return fused_save_from(st, B, T, H, r, k, v, w, u, nullptr, gate, gn_scale, gn_offset, gn_eps, out, y, stats, saved_states);
}

// ------------------------------------------------------------------------------------------
// Long sequences, few pairs: time cut into segments that run side by side.
//
// With fewer (batch, head) pairs than half the compute units most of the chip would idle while each
// pair walks its sequence alone.  The map from a segment's incoming state to its outgoing state is
// affine, S_out = D o S_in + U with D[j] = exp(-sum_t exp(w_t[j])) over the segment and U the state
// the segment builds from zero, so: (A) every segment runs from a zero state (all segments at once;
// a (B,T,C) tensor cut into P equal segments IS a (B*P, T/P, C) tensor; no y in this pass) and leaves
// U and, from the producer waves, the exponent of D; (B) a tiny kernel chains the P affine maps per pair,
// leaving each segment's true incoming state where its U was (and the final state); (C) every
// segment runs again from its true state and writes y.  Twice the forward work on P times the
// workgroups.
// ------------------------------------------------------------------------------------------
// kReverse: the same chain walked from the last segment to the first, which is what the reverse
// state of the backward pass obeys (the gradient arriving at the end of segment p is what segment
// p + 1 sends into its incoming state: its own contribution plus D_{p+1} times what arrives at its end).
template <typename Ts, bool kReverse, int P>
__global__ __launch_bounds__(256) void segment_chain_kernel(int H, const Ts *__restrict__ s0, const int64_t *__restrict__ map,
                                                            const float *__restrict__ dsum, float *__restrict__ states, Ts *__restrict__ sT,
                                                            float *__restrict__ sT32)   // the final state: as Ts and / or as fp32 (either may be null)
{
    // Thread: four value columns i0..i0+3 of one key row j of one (batch, head): 1024 threads per pair,
    // gridDim.x * 256 = B * H * 1024.  states[(b*P + seg), h] holds U on entry and the segment's
    // incoming state on exit.  All P loads are issued before the chain is walked (their addresses do
    // not depend on it): the kernel takes about two memory round trips instead of 2 P.
    const int e = blockIdx.x * 256 + threadIdx.x;
    const int i0 = (e & 15) * 4, j = (e >> 4) & 63, bh = e >> 10;
    const int b = bh / H, h = bh - b * H;
    const int64_t np = (int64_t)(gridDim.x >> 2) * P;   // pairs of all segments
    auto pair_of_step = [&](int n) { return ((int64_t)b * P + (kReverse ? P - 1 - n : n)) * H + h; };   // step n of the walk
    float4 x[P];
    float d[P];
#pragma unroll
    for (int n = 0; n < P; ++n) {
        const int64_t vp = pair_of_step(n);
        x[n] = *reinterpret_cast<const float4 *>(states + (vp * kN + j) * kN + i0);
        d[n] = (dsum[vp * kN + j] + dsum[(np + vp) * kN + j]) + (dsum[(2 * np + vp) * kN + j] + dsum[(3 * np + vp) * kN + j]);
    }
    float S[4] = {0.f, 0.f, 0.f, 0.f};
    if (s0) {
        const int64_t row = map ? map[b] : (int64_t)b;
        load4(s0 + ((row * H + h) * kN + j) * kN + i0, S);
    }
#pragma unroll
    for (int n = 0; n < P; ++n) {
        const float dd = exp2_fast(-d[n]);
        *reinterpret_cast<float4 *>(states + (pair_of_step(n) * kN + j) * kN + i0) = make_float4(S[0], S[1], S[2], S[3]);
        S[0] = fmaf(S[0], dd, x[n].x); S[1] = fmaf(S[1], dd, x[n].y); S[2] = fmaf(S[2], dd, x[n].z); S[3] = fmaf(S[3], dd, x[n].w);
    }
    if (sT) store4(sT + (((int64_t)b * H + h) * kN + j) * kN + i0, S[0], S[1], S[2], S[3]);
    if (sT32) store4(sT32 + (((int64_t)b * H + h) * kN + j) * kN + i0, S[0], S[1], S[2], S[3]);
}
template <typename Ts, bool kReverse>
static hipError_t launch_chain(hipStream_t st, int P, int64_t B, int64_t H, const Ts *s0, const int64_t *map,
                               const float *dsum, float *states, Ts *sT, float *sT32 = nullptr)
{
    const dim3 grid((unsigned)(B * H * 4)), block(256);
    switch (P) {
    case 2: hipLaunchKernelGGL((segment_chain_kernel<Ts, kReverse, 2>), grid, block, 0, st, (int)H, s0, map, dsum, states, sT, sT32); break;
    case 4: hipLaunchKernelGGL((segment_chain_kernel<Ts, kReverse, 4>), grid, block, 0, st, (int)H, s0, map, dsum, states, sT, sT32); break;
    case 8: hipLaunchKernelGGL((segment_chain_kernel<Ts, kReverse, 8>), grid, block, 0, st, (int)H, s0, map, dsum, states, sT, sT32); break;
    case 16: hipLaunchKernelGGL((segment_chain_kernel<Ts, kReverse, 16>), grid, block, 0, st, (int)H, s0, map, dsum, states, sT, sT32); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Number of segments for this shape (1 = not worth it / not possible) and their length: the pairs
// times the segments should still fit the chip once, a segment is a whole number of chunks and at
// least four of them.  A single sequence need not divide evenly: what is left over behind the P
// segments (less than P chunks) follows as an ordinary pass from the state the segments end in.
// (With B > 1 the first P * L tokens of every batch row are not one contiguous (B*P, L, C) tensor.)
static int forward_segments_plan(int64_t B, int64_t T, int64_t H, int64_t *L) {
    const int64_t pairs = B * H, cus = compute_units();
    // (two passes over T / P tokens and two more launches against one pass over T: nothing to gain
    // below four segments or on short sequences)
    if (T < 1024) return 1;
    for (int P = 16; P >= 4; P >>= 1) {
        const int64_t l = T / P / CL * CL;
        if (pairs * P > cus || l < 4 * CL) continue;
        if (P * l != T && B != 1) continue;
        *L = l;
        return P;
    }
    return 1;
}
int chunk_forward_segments(int64_t B, int64_t T, int64_t H) {
    int64_t L;
    return forward_segments_plan(B, T, H, &L);
}
int64_t chunk_forward_segments_remainder(int64_t B, int64_t T, int64_t H) {
    int64_t L = 0;
    const int P = forward_segments_plan(B, T, H, &L);
    return P <= 1 ? 0 : T - P * L;
}
size_t chunk_forward_segments_workspace_bytes(int64_t B, int64_t T, int64_t H) {
    const int P = chunk_forward_segments(B, T, H);
    // per segment and pair a state and the decay exponents; per pair the state the segments end in
    return P <= 1 ? 0 : ((size_t)(B * P * H) * (kN * kN + 4 * kN) + (size_t)(B * H) * kN * kN) * sizeof(float);
}

// A remainder needs fp32 states at the boundary or no final state (see the API layer's check).
// With `gate` the passes that produce output run the fused output stage (y = out then).
hipError_t chunk_forward_segments_run(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                                      const void *r, const void *k, const void *v, const void *w, const void *u,
                                      const void *s0, const int64_t *map, void *y, void *sT, void *workspace,
                                      const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps)
{
    int64_t L = 0;
    const int P = forward_segments_plan(B, T, H, &L);
    const int64_t rows = B * P, rem = T - P * L;
    float *states = (float *)workspace, *dsum = states + rows * H * kN * kN, *mid = dsum + rows * H * 4 * kN;
    hipError_t e = chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, nullptr, nullptr, nullptr, states, nullptr, dsum);
    if (e != hipSuccess) return e;
    void *end_state = rem ? nullptr : sT;   // with a remainder the segments end in `mid`
    e = state_dtype == kF32 ? launch_chain<float, false>(st, P, B, H, (const float *)s0, map, dsum, states, (float *)end_state, rem ? mid : nullptr)
                            : launch_chain<bf16_t, false>(st, P, B, H, (const bf16_t *)s0, map, dsum, states, (bf16_t *)end_state, rem ? mid : nullptr);
    if (e != hipSuccess) return e;
    e = gate ? chunk_forward_fused(st, kF32, rows, L, H, r, k, v, w, u, states, nullptr, gate, gn_scale, gn_offset, gn_eps, y, nullptr)
             : chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, states, nullptr, y, nullptr, nullptr);
    if (e != hipSuccess || rem == 0) return e;
    const int64_t off = P * L * H * kN;   // (B == 1) elements in front of the remainder
    auto at = [&](const void *p) { return (const void *)((const bf16_t *)p + off); };
    if (gate)
        return chunk_forward_fused(st, kF32, B, rem, H, at(r), at(k), at(v), at(w), u, mid, nullptr, at(gate), gn_scale, gn_offset, gn_eps,
                                   (bf16_t *)y + off, sT);
    return chunk_forward(st, kF32, B, rem, H, at(r), at(k), at(v), at(w), u, mid, nullptr, (bf16_t *)y + off, sT, nullptr);
}

hipError_t segment_chain_reverse(hipStream_t st, int P, int64_t B, int64_t H, const float *dsum, float *states,
                                 const float *arriving, float *leaving) {
    return launch_chain<float, true>(st, P, B, H, arriving, nullptr, dsum, states, leaving);
}
hipError_t segment_chain_forward(hipStream_t st, int P, int64_t B, int64_t H, const float *dsum, float *states, const float *s0) {
    return launch_chain<float, false>(st, P, B, H, s0, nullptr, dsum, states, nullptr);
}

// ------------------------------------------------------------------------------------------
// The same for the training pair (saving forward, backward from the saved states): the forward
// keeps every segment's incoming state and decay exponents for the backward, whose reverse state
// is chained the same way (see chunk_backward_saved_segments).
// ------------------------------------------------------------------------------------------
int chunk_train_segments(int64_t B, int64_t T, int64_t H) {
    const int64_t pairs = B * H, cus = compute_units();
    // (two state-only passes at 0.7 of a forward each on top of the forward and the backward: 1.5
    // times the work on P times the workgroups, and three small kernels)
    if (T < 1024) return 1;
    for (int P = 16; P >= 2; P >>= 1)
        if (pairs * P <= cus && T % (P * CL) == 0 && T / P >= 4 * CL && (T >= 2048 || P >= 4)) return P;
    return 1;
}
TrainSegments train_segments_layout(int64_t B, int64_t T, int64_t H, void *extra) {
    TrainSegments s;
    s.P = chunk_train_segments(B, T, H);
    const size_t pairs = (size_t)(B * s.P * H);
    s.states = reinterpret_cast<float *>(extra);
    s.dsum = s.states + pairs * kN * kN;
    s.gstates = s.dsum + pairs * 4 * kN;
    s.gu_rows = s.gstates + pairs * kN * kN;
    s.bytes = (pairs * (2 * kN * kN + 4 * kN) + (size_t)(B * s.P * H) * kN) * sizeof(float);   // (gu rows: room for fp32)
    return s;
}

hipError_t chunk_forward_save_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                       const void *r, const void *k, const void *v, const void *w, const void *u,
                                       void *y, void *saved, void *extra)
{
    const TrainSegments s = train_segments_layout(B, T, H, extra);
    const int64_t L = T / s.P, rows = B * s.P;
    hipError_t e = chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, nullptr, nullptr, nullptr, s.states, nullptr, s.dsum);
    if (e != hipSuccess) return e;
    if ((e = launch_chain<float, false>(st, s.P, B, H, nullptr, nullptr, s.dsum, s.states, nullptr)) != hipSuccess) return e;
    return chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, s.states, nullptr, y, nullptr, saved);
}

// The same with the fused output stage in the second pass.  out, y, gate and the statistics are indexed by
// token, and the tokens of the (B*P, T/P) rows are those of the (B, T) rows in the same order.
hipError_t chunk_forward_fused_save_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                             const void *r, const void *k, const void *v, const void *w, const void *u,
                                             const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                                             void *out, void *y, float *stats, void *saved, void *extra)
{
    const TrainSegments s = train_segments_layout(B, T, H, extra);
    const int64_t L = T / s.P, rows = B * s.P;
    hipError_t e = chunk_forward(st, kF32, rows, L, H, r, k, v, w, u, nullptr, nullptr, nullptr, s.states, nullptr, s.dsum);
    if (e != hipSuccess) return e;
    if ((e = launch_chain<float, false>(st, s.P, B, H, nullptr, nullptr, s.dsum, s.states, nullptr)) != hipSuccess) return e;
    return fused_save_from(st, rows, L, H, r, k, v, w, u, s.states, gate, gn_scale, gn_offset, gn_eps, out, y, stats, saved);
}

}  // namespace wkv6
