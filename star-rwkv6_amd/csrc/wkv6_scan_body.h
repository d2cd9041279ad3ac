// Per-timestep WKV6 recurrence for one (batch, head) pair, as device functions over a caller-
// provided LDS block: used by the stand-alone scan kernels (wkv6_scan.hip) and, as the exact second
// pass of a workgroup whose decay left the representable range, inside the chunked kernels
// (wkv6_chunk.hip).
#pragma once
#include "wkv6_common.h"

namespace wkv6 {

constexpr int TC = 16;  // timesteps per LDS tile

__device__ __forceinline__ float sum8_lanes(float x) {
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    x += __shfl_xor(x, 4);
    return x;
}

__device__ __forceinline__ void lds_store8(float *p, const float (&f)[8]) {
    *reinterpret_cast<float4 *>(p) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4 *>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}

// ------------------------------------------------------------------------------------------
// Forward.  wave q of NW owns key rows j in [64/NW q, 64/NW (q+1)); lane i owns value column i.
//   y_t[i]  = v_t[i] * sum_j r_t[j] u[j] k_t[j]  +  sum_j r_t[j] S[j][i]
//   S[j][i] = S[j][i] * d_t[j] + k_t[j] v_t[i]
// ------------------------------------------------------------------------------------------
template <int NW> struct alignas(16) ScanFwdLdsT {
    float s_r[TC][kN], s_k[TC][kN], s_d[TC][kN], s_v[TC][kN];
    float s_part[NW][TC][kN];
    float s_ruk[TC];
    float s_u[kN];
};
typedef ScanFwdLdsT<4> ScanFwdLds;

// Work of one (b, h) pair by the first NW waves of the workgroup (wave q owns key rows
// [64/NW * q, 64/NW * (q+1)); the first 256 threads also stage the tiles and fold the partials);
// further threads only keep the barriers company (the chunked kernels call this with NW = 4 and 768 threads).
template <typename Tin, typename Tout, typename Ts, int NW = 4>
__device__ __forceinline__ void scan_fwd_body(ScanFwdLdsT<NW> &L, int b, int h, int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u,
        const Ts *__restrict__ s0, const int64_t *__restrict__ map,
        Tout *__restrict__ y, Ts *__restrict__ sT, bool reverse = false)   // reverse: timestep t reads row T-1-t (no y then)
{
    auto &s_r = L.s_r; auto &s_k = L.s_k; auto &s_d = L.s_d; auto &s_v = L.s_v;
    auto &s_part = L.s_part; auto &s_ruk = L.s_ruk; auto &s_u = L.s_u;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6;
    constexpr int RW = kN / NW;   // key rows per wave
    if (tid >= 64 * NW) {   // same barrier sequence as below, no work
        __syncthreads();
        for (int t0 = 0; t0 < T; t0 += TC) { __syncthreads(); __syncthreads(); }
        return;
    }
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;

    // staging role: threads 0..127 bring r,k ; 128..255 bring v,w ; 8 channels of one timestep each
    const int half = tid >> 7, st = (tid & 127) >> 3, sc = (tid & 7) * 8;
    const Tin *pa = (half == 0 ? r : v) + base + sc;
    const Tin *pb = (half == 0 ? k : w) + base + sc;
    Raw8<Tin> ra, rb;

    float s[RW];
    if (s0 != nullptr) {
        const int64_t row = map ? map[b] : (int64_t)b;
        const Ts *p = s0 + ((row * H + h) * kN + RW * q) * kN + lane;
#pragma unroll
        for (int jj = 0; jj < RW; ++jj) s[jj] = load1(p + jj * kN);
    } else {
#pragma unroll
        for (int jj = 0; jj < RW; ++jj) s[jj] = 0.f;
    }
    if (tid < kN) s_u[tid] = load1(u + h * kN + tid);

    auto prefetch = [&](int t0) {
        const int t = t0 + st;
        if (tid >= 256) return;
        if (t < T) { const int64_t row = reverse ? T - 1 - t : t; ra.load(pa + row * C); rb.load(pb + row * C); }
        else { ra.zero(); rb.zero(); }
    };
    prefetch(0);
    __syncthreads();

    for (int t0 = 0; t0 < T; t0 += TC) {
        if (tid < 256) {   // registers -> LDS tile
            float fa[8], fb[8];
            ra.to_float(fa); rb.to_float(fb);
            if (half == 0) {
                lds_store8(&s_r[st][sc], fa);
                lds_store8(&s_k[st][sc], fb);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) p = fmaf(fa[i] * fb[i], s_u[sc + i], p);
                p = sum8_lanes(p);
                if ((tid & 7) == 0) s_ruk[st] = p;
            } else {
                lds_store8(&s_v[st][sc], fa);
#pragma unroll
                for (int i = 0; i < 8; ++i) fb[i] = decay_from_raw(fb[i]);
                lds_store8(&s_d[st][sc], fb);
            }
        }
        __syncthreads();
        prefetch(t0 + TC);
        const int nt = min(TC, T - t0);
        for (int t = 0; t < nt; ++t) {
            float rr[RW], kk[RW], dd[RW];
#pragma unroll
            for (int g = 0; g < RW / 4; ++g) {
                const float4 a = *reinterpret_cast<const float4 *>(&s_r[t][RW * q + 4 * g]);
                const float4 c = *reinterpret_cast<const float4 *>(&s_k[t][RW * q + 4 * g]);
                const float4 e = *reinterpret_cast<const float4 *>(&s_d[t][RW * q + 4 * g]);
                rr[4 * g] = a.x; rr[4 * g + 1] = a.y; rr[4 * g + 2] = a.z; rr[4 * g + 3] = a.w;
                kk[4 * g] = c.x; kk[4 * g + 1] = c.y; kk[4 * g + 2] = c.z; kk[4 * g + 3] = c.w;
                dd[4 * g] = e.x; dd[4 * g + 1] = e.y; dd[4 * g + 2] = e.z; dd[4 * g + 3] = e.w;
            }
            const float vi = s_v[t][lane];
            float acc0 = (q == 0) ? vi * s_ruk[t] : 0.f, acc1 = 0.f;
#pragma unroll
            for (int jj = 0; jj < RW; jj += 2) {
                const float x0 = kk[jj] * vi, x1 = kk[jj + 1] * vi;
                acc0 = fmaf(rr[jj], s[jj], acc0);
                acc1 = fmaf(rr[jj + 1], s[jj + 1], acc1);
                s[jj] = fmaf(s[jj], dd[jj], x0);
                s[jj + 1] = fmaf(s[jj + 1], dd[jj + 1], x1);
            }
            s_part[q][t][lane] = acc0 + acc1;
        }
        __syncthreads();
        {   // sum the four wave partials, one rounding, coalesced store
            const int t = tid >> 4, c4 = (tid & 15) * 4;
            if (t < nt && tid < 256) {
                float4 a = *reinterpret_cast<const float4 *>(&s_part[0][t][c4]);
#pragma unroll
                for (int qq = 1; qq < NW; ++qq) {
                    const float4 c = *reinterpret_cast<const float4 *>(&s_part[qq][t][c4]);
                    a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
                }
                if (y) store4(y + base + (int64_t)(t0 + t) * C + c4, a.x, a.y, a.z, a.w);
            }
        }
        // the next tile's LDS writes touch s_r/s_k/s_v/s_d/s_ruk only, all readers of which are
        // past the barrier above; s_part is rewritten only after the barrier that follows them.
    }
    if (sT != nullptr) {
        Ts *p = sT + (((int64_t)b * H + h) * kN + RW * q) * kN + lane;
#pragma unroll
        for (int jj = 0; jj < RW; ++jj) store1(p + jj * kN, s[jj]);
    }
}

// ------------------------------------------------------------------------------------------
// Backward, sweep A (time ascending): gr, gu partials and P_t[j] = r_t[j] * gr'_t[j] (fp32
// workspace), where gr'_t[j] = sum_i gy_t[i] S_t[j][i] is gr without the u term.
// lane j owns key row j; wave q owns value columns [16q,16q+16).
// ------------------------------------------------------------------------------------------
template <int NW> struct alignas(16) ScanBwdALdsT {
    float s_r[TC][kN], s_k[TC][kN], s_d[TC][kN], s_v[TC][kN], s_g[TC][kN];
    float s_part[NW][TC][kN];
    float s_vgy[TC];
    float s_u[kN];
};
typedef ScanBwdALdsT<4> ScanBwdALds;

// P is addressed as wsP[t * pstride + channel-in-head]: the caller points wsP at this head's
// first element ((B,T,C) layout: pstride = C; a private [T][64] block: pstride = 64).
// The first NW waves work (wave q owns value columns [64/NW q, 64/NW (q+1)); NW <= 16; the first
// 256 threads also stage the tiles and finish the rows); further threads only keep the barriers company.
template <typename Tin, typename Tout, int NW = 4>
__device__ __forceinline__ void scan_bwd_a_body(ScanBwdALdsT<NW> &L, int b, int h, int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u, const Tout *__restrict__ gy,
        Tout *__restrict__ gr, Tout *__restrict__ gu, float *__restrict__ wsP, int64_t pstride,
        const float *__restrict__ s0 = nullptr, const float *__restrict__ gsT = nullptr, float *fT = nullptr)
{
    // State gradients (all three null for the stateless operator): s0 = this pair's initial state
    // [key][value] fp32; gsT = the gradient arriving at its final state; fT[64] receives
    // F_T[j] = sum_i S_T[j][i] gsT[j][i], the anchor of the gw suffix sums of sweep B.
    auto &s_r = L.s_r; auto &s_k = L.s_k; auto &s_d = L.s_d; auto &s_v = L.s_v; auto &s_g = L.s_g;
    auto &s_part = L.s_part; auto &s_vgy = L.s_vgy; auto &s_u = L.s_u;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6;
    constexpr int RW = kN / NW;   // value columns per wave
    const bool first256 = tid < 256;
    if (tid >= 64 * NW) {   // same barrier sequence as below, no work
        __syncthreads();
        for (int t0 = 0; t0 < T; t0 += TC) { __syncthreads(); __syncthreads(); __syncthreads(); }
        __syncthreads();
        return;
    }
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;

    // staging: threads 0..127 bring v,gy ; 128..255 bring k,w,r
    const int half = tid >> 7, st = (tid & 127) >> 3, sc = (tid & 7) * 8;
    Raw8<Tin> ra, rb, rc;
    Raw8<Tout> rg;

    float s[RW];
#pragma unroll
    for (int ii = 0; ii < RW; ++ii) s[ii] = s0 ? s0[lane * kN + RW * q + ii] : 0.f;
    if (tid < kN) s_u[tid] = load1(u + h * kN + tid);
    float gu_acc[4] = {0.f, 0.f, 0.f, 0.f};

    auto prefetch = [&](int t0) {
        const int t = t0 + st;
        const int64_t o = base + (int64_t)t * C + sc;
        if (!first256) return;
        if (t < T) {
            if (half == 0) { ra.load(v + o); rg.load(gy + o); }
            else { ra.load(k + o); rb.load(w + o); rc.load(r + o); }
        } else { ra.zero(); rb.zero(); rc.zero(); rg.zero(); }
    };
    prefetch(0);
    __syncthreads();

    for (int t0 = 0; t0 < T; t0 += TC) {
        if (first256) {
            float fa[8], fb[8];
            ra.to_float(fa);
            if (half == 0) {
                rg.to_float(fb);
                lds_store8(&s_v[st][sc], fa);
                lds_store8(&s_g[st][sc], fb);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) p = fmaf(fa[i], fb[i], p);
                p = sum8_lanes(p);
                if ((tid & 7) == 0) s_vgy[st] = p;
            } else {
                lds_store8(&s_k[st][sc], fa);
                rb.to_float(fb);
#pragma unroll
                for (int i = 0; i < 8; ++i) fb[i] = decay_from_raw(fb[i]);
                lds_store8(&s_d[st][sc], fb);
                rc.to_float(fb);
                lds_store8(&s_r[st][sc], fb);
            }
        }
        __syncthreads();
        prefetch(t0 + TC);
        const int nt = min(TC, T - t0);
        for (int t = 0; t < nt; ++t) {
            float vv[RW], gg[RW];
#pragma unroll
            for (int g = 0; g < RW / 4; ++g) {
                const float4 a = *reinterpret_cast<const float4 *>(&s_v[t][RW * q + 4 * g]);
                const float4 c = *reinterpret_cast<const float4 *>(&s_g[t][RW * q + 4 * g]);
                vv[4 * g] = a.x; vv[4 * g + 1] = a.y; vv[4 * g + 2] = a.z; vv[4 * g + 3] = a.w;
                gg[4 * g] = c.x; gg[4 * g + 1] = c.y; gg[4 * g + 2] = c.z; gg[4 * g + 3] = c.w;
            }
            const float kj = s_k[t][lane], dj = s_d[t][lane];
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int ii = 0; ii < RW; ii += 2) {
                const float x0 = kj * vv[ii], x1 = kj * vv[ii + 1];
                acc0 = fmaf(gg[ii], s[ii], acc0);
                acc1 = fmaf(gg[ii + 1], s[ii + 1], acc1);
                s[ii] = fmaf(s[ii], dj, x0);
                s[ii + 1] = fmaf(s[ii + 1], dj, x1);
            }
            s_part[q][t][lane] = acc0 + acc1;
        }
        __syncthreads();
        {
            const int t = tid >> 4, c4 = (tid & 15) * 4;
            if (t < nt && first256) {
                float4 a = *reinterpret_cast<const float4 *>(&s_part[0][t][c4]);
#pragma unroll
                for (int qq = 1; qq < NW; ++qq) {
                    const float4 c = *reinterpret_cast<const float4 *>(&s_part[qq][t][c4]);
                    a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
                }
                const float4 r4 = *reinterpret_cast<const float4 *>(&s_r[t][c4]);
                const float4 k4 = *reinterpret_cast<const float4 *>(&s_k[t][c4]);
                const float4 u4 = *reinterpret_cast<const float4 *>(&s_u[c4]);
                const float vg = s_vgy[t];
                const int64_t o = base + (int64_t)(t0 + t) * C + c4;
                store4(gr + o, fmaf(u4.x * k4.x, vg, a.x), fmaf(u4.y * k4.y, vg, a.y),
                       fmaf(u4.z * k4.z, vg, a.z), fmaf(u4.w * k4.w, vg, a.w));
                *reinterpret_cast<float4 *>(wsP + (int64_t)(t0 + t) * pstride + c4) =
                    make_float4(r4.x * a.x, r4.y * a.y, r4.z * a.z, r4.w * a.w);
                gu_acc[0] = fmaf(r4.x * k4.x, vg, gu_acc[0]);
                gu_acc[1] = fmaf(r4.y * k4.y, vg, gu_acc[1]);
                gu_acc[2] = fmaf(r4.z * k4.z, vg, gu_acc[2]);
                gu_acc[3] = fmaf(r4.w * k4.w, vg, gu_acc[3]);
            }
        }
        __syncthreads();  // finalisers read s_r/s_k/s_vgy; the next tile's staging overwrites them
    }
    // gu: the 16 threads with equal (tid & 15) hold partial sums of the same 4 channels over
    // different timesteps.  Lanes l, l^16, l^32, l^48 fold with wavefront shuffles, the four waves
    // through LDS -- no atomics.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        gu_acc[i] += __shfl_xor(gu_acc[i], 16);
        gu_acc[i] += __shfl_xor(gu_acc[i], 32);
    }
    if (lane < 16 && first256) {   // (the finishing threads: waves 0..3)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_part[0][q][lane * 4 + i] = gu_acc[i];
    }
    if (fT) {   // s now holds S_T
        float f = 0.f;
#pragma unroll
        for (int ii = 0; ii < RW; ++ii) f = fmaf(s[ii], gsT ? gsT[lane * kN + RW * q + ii] : 0.f, f);
        s_part[1][q][lane] = f;
    }
    __syncthreads();
    if (tid < kN) {
        const float g = s_part[0][0][tid] + s_part[0][1][tid] + s_part[0][2][tid] + s_part[0][3][tid];
        store1(gu + (int64_t)b * C + h * kN + tid, g);
        if (fT) {
            float f = 0.f;
#pragma unroll
            for (int qq = 0; qq < NW; ++qq) f += s_part[1][qq][tid];
            fT[tid] = f;
        }
    }
}

// ------------------------------------------------------------------------------------------
// Backward, sweep B (time descending): gk, gv, gw.  Reverse state
//   G[j][i] <- r_t[j] gy_t[i] + d_t[j] G[j][i]          (holds G_{t+1} when step t reads it)
// is kept twice: waves 0..3 ("K role") with lane = key row j for gk_t[j] = sum_i v_t[i] G[j][i],
// waves 4..7 ("V role") with lane = value column i for gv_t[i] = sum_j k_t[j] G[j][i], so neither
// needs a cross-lane reduction per timestep.
// gw uses the flow-balance identity (same quantity as the reference's running sums,
// rwkv_kernels.cu:358-405):   gw_t[j] = -exp(w_t[j]) * ( sum_{m>t} P_m[j] - sum_{m>=t} Q_m[j] ),
// Q_m[j] = k_m[j] gk'_m[j], P from sweep A; accumulated as one running difference per channel.
// ------------------------------------------------------------------------------------------
template <int NWR> struct alignas(16) ScanBwdBLdsT {
    float s_r[TC][kN], s_k[TC][kN], s_d[TC][kN], s_v[TC][kN], s_g[TC][kN];
    float s_pk[NWR][TC][kN], s_pv[NWR][TC][kN];
    float s_e[TC][kN];
    float s_vgy[TC], s_ruk[TC];
    float s_u[kN];
};
typedef ScanBwdBLdsT<4> ScanBwdBLds;

// The first 2 NWR waves of the workgroup work: NWR in the K role, then NWR in the V role, each
// owning 64/NWR value columns / key rows; the first 512 threads also stage the tiles and finish the
// rows.  P addressed as in sweep A.
template <typename Tin, typename Tout, int NWR = 4>
__device__ __forceinline__ void scan_bwd_b_body(ScanBwdBLdsT<NWR> &L, int b, int h, int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u, const Tout *__restrict__ gy,
        const float *__restrict__ wsP, int64_t pstride,
        Tout *__restrict__ gk, Tout *__restrict__ gv, Tout *__restrict__ gw,
        const float *__restrict__ gsT = nullptr, const float *fT = nullptr, float *__restrict__ gs0 = nullptr,
        bool first_decay_unused = true)
{
    // State gradients (null / true for the stateless operator): the reverse state starts from gsT
    // (this pair's [key][value] fp32 block) and ends as gs0 = dL/dS_0; fT[64] anchors the gw suffix
    // sums (sweep A); first_decay_unused = the initial state is zero, so d_0 reaches no output.
    auto &s_r = L.s_r; auto &s_k = L.s_k; auto &s_d = L.s_d; auto &s_v = L.s_v; auto &s_g = L.s_g;
    auto &s_pk = L.s_pk; auto &s_pv = L.s_pv; auto &s_e = L.s_e;
    auto &s_vgy = L.s_vgy; auto &s_ruk = L.s_ruk; auto &s_u = L.s_u;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int RW = kN / NWR;
    if (tid >= 128 * NWR) {   // a larger workgroup: same barrier sequence as below, no work
        __syncthreads();
        for (int t0 = ((T - 1) / TC) * TC; t0 >= 0; t0 -= TC) { __syncthreads(); __syncthreads(); __syncthreads(); }
        return;
    }
    const int q = wave % NWR;
    const bool role_k = wave < NWR;
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;

    // staging: group 0 brings r,k ; 1 brings v,gy ; 2 brings w ; 3 idles.  The finaliser threads
    // (tid < 256, 4 channels of one timestep) additionally hold P and raw w of their own element.
    const int grp = tid >> 7, st = (tid & 127) >> 3, sc = (tid & 7) * 8;
    const int ft = (tid & 255) >> 4, fc = (tid & 15) * 4;
    Raw8<Tin> ra, rb;
    Raw8<Tout> rg;
    float4 preP = make_float4(0, 0, 0, 0), curP;
    float preW[4] = {0, 0, 0, 0}, curW[4];

    float g[RW];
#pragma unroll
    for (int i = 0; i < RW; ++i)
        g[i] = !gsT ? 0.f : role_k ? gsT[lane * kN + RW * q + i] : gsT[(RW * q + i) * kN + lane];
    if (tid < kN) s_u[tid] = load1(u + h * kN + tid);
    float carry[4] = {0.f, 0.f, 0.f, 0.f};  // sum over later tiles of (P - Q), finaliser channels
    if (fT && tid < 256) {
#pragma unroll
        for (int i = 0; i < 4; ++i) carry[i] = fT[fc + i];
    }

    auto prefetch = [&](int t0) {
        const int t = t0 + st;
        const int64_t o = base + (int64_t)t * C + sc;
        const bool ok = (t0 >= 0) && (t < T);
        if (ok) {
            if (grp == 0) { ra.load(r + o); rb.load(k + o); }
            else if (grp == 1) { ra.load(v + o); rg.load(gy + o); }
            else if (grp == 2) { ra.load(w + o); }
        } else { ra.zero(); rb.zero(); rg.zero(); }
        if (tid < 256) {
            const int tf = t0 + ft;
            if (t0 >= 0 && tf < T) {
                const int64_t of = base + (int64_t)tf * C + fc;
                preP = *reinterpret_cast<const float4 *>(wsP + (int64_t)tf * pstride + fc);
#pragma unroll
                for (int i = 0; i < 4; ++i) preW[i] = load1(w + of + i);
            }
        }
    };
    const int last_t0 = ((T - 1) / TC) * TC;
    prefetch(last_t0);
    __syncthreads();

    for (int t0 = last_t0; t0 >= 0; t0 -= TC) {
        {
            float fa[8], fb[8];
            ra.to_float(fa);
            if (grp == 0) {
                rb.to_float(fb);
                lds_store8(&s_r[st][sc], fa);
                lds_store8(&s_k[st][sc], fb);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) p = fmaf(fa[i] * fb[i], s_u[sc + i], p);
                p = sum8_lanes(p);
                if ((tid & 7) == 0) s_ruk[st] = p;
            } else if (grp == 1) {
                rg.to_float(fb);
                lds_store8(&s_v[st][sc], fa);
                lds_store8(&s_g[st][sc], fb);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) p = fmaf(fa[i], fb[i], p);
                p = sum8_lanes(p);
                if ((tid & 7) == 0) s_vgy[st] = p;
            } else if (grp == 2) {
#pragma unroll
                for (int i = 0; i < 8; ++i) fa[i] = decay_from_raw(fa[i]);
                lds_store8(&s_d[st][sc], fa);
            }
            curP = preP;
#pragma unroll
            for (int i = 0; i < 4; ++i) curW[i] = preW[i];
        }
        __syncthreads();
        prefetch(t0 - TC);
        const int nt = min(TC, T - t0);
        if (role_k) {
            for (int t = nt - 1; t >= 0; --t) {
                float vv[RW], gg[RW];
#pragma unroll
                for (int a4 = 0; a4 < RW / 4; ++a4) {
                    const float4 a = *reinterpret_cast<const float4 *>(&s_v[t][RW * q + 4 * a4]);
                    const float4 c = *reinterpret_cast<const float4 *>(&s_g[t][RW * q + 4 * a4]);
                    vv[4 * a4] = a.x; vv[4 * a4 + 1] = a.y; vv[4 * a4 + 2] = a.z; vv[4 * a4 + 3] = a.w;
                    gg[4 * a4] = c.x; gg[4 * a4 + 1] = c.y; gg[4 * a4 + 2] = c.z; gg[4 * a4 + 3] = c.w;
                }
                const float rj = s_r[t][lane], dj = s_d[t][lane];
                float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
                for (int ii = 0; ii < RW; ii += 2) {
                    acc0 = fmaf(vv[ii], g[ii], acc0);
                    acc1 = fmaf(vv[ii + 1], g[ii + 1], acc1);
                    g[ii] = fmaf(g[ii], dj, rj * gg[ii]);
                    g[ii + 1] = fmaf(g[ii + 1], dj, rj * gg[ii + 1]);
                }
                s_pk[q][t][lane] = acc0 + acc1;
            }
        } else {
            for (int t = nt - 1; t >= 0; --t) {
                float rr[RW], kk[RW], dd[RW];
#pragma unroll
                for (int a4 = 0; a4 < RW / 4; ++a4) {
                    const float4 a = *reinterpret_cast<const float4 *>(&s_r[t][RW * q + 4 * a4]);
                    const float4 c = *reinterpret_cast<const float4 *>(&s_k[t][RW * q + 4 * a4]);
                    const float4 e = *reinterpret_cast<const float4 *>(&s_d[t][RW * q + 4 * a4]);
                    rr[4 * a4] = a.x; rr[4 * a4 + 1] = a.y; rr[4 * a4 + 2] = a.z; rr[4 * a4 + 3] = a.w;
                    kk[4 * a4] = c.x; kk[4 * a4 + 1] = c.y; kk[4 * a4 + 2] = c.z; kk[4 * a4 + 3] = c.w;
                    dd[4 * a4] = e.x; dd[4 * a4 + 1] = e.y; dd[4 * a4 + 2] = e.z; dd[4 * a4 + 3] = e.w;
                }
                const float gi = s_g[t][lane];
                float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
                for (int jj = 0; jj < RW; jj += 2) {
                    acc0 = fmaf(kk[jj], g[jj], acc0);
                    acc1 = fmaf(kk[jj + 1], g[jj + 1], acc1);
                    g[jj] = fmaf(g[jj], dd[jj], rr[jj] * gi);
                    g[jj + 1] = fmaf(g[jj + 1], dd[jj + 1], rr[jj + 1] * gi);
                }
                s_pv[q][t][lane] = acc0 + acc1;
            }
        }
        __syncthreads();
        float Qv[4] = {0.f, 0.f, 0.f, 0.f};
        const int64_t of = base + (int64_t)(t0 + ft) * C + fc;
        if (tid < 256) {            // gk, and E = P - Q for the gw suffix sums
            float e[4] = {0.f, 0.f, 0.f, 0.f};
            if (ft < nt) {
                float4 a = *reinterpret_cast<const float4 *>(&s_pk[0][ft][fc]);
#pragma unroll
                for (int qq = 1; qq < NWR; ++qq) {
                    const float4 c = *reinterpret_cast<const float4 *>(&s_pk[qq][ft][fc]);
                    a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
                }
                const float4 r4 = *reinterpret_cast<const float4 *>(&s_r[ft][fc]);
                const float4 k4 = *reinterpret_cast<const float4 *>(&s_k[ft][fc]);
                const float4 u4 = *reinterpret_cast<const float4 *>(&s_u[fc]);
                const float vg = s_vgy[ft];
                store4(gk + of, fmaf(u4.x * r4.x, vg, a.x), fmaf(u4.y * r4.y, vg, a.y),
                       fmaf(u4.z * r4.z, vg, a.z), fmaf(u4.w * r4.w, vg, a.w));
                Qv[0] = k4.x * a.x; Qv[1] = k4.y * a.y; Qv[2] = k4.z * a.z; Qv[3] = k4.w * a.w;
                e[0] = curP.x - Qv[0]; e[1] = curP.y - Qv[1]; e[2] = curP.z - Qv[2]; e[3] = curP.w - Qv[3];
            }
            *reinterpret_cast<float4 *>(&s_e[ft][fc]) = make_float4(e[0], e[1], e[2], e[3]);
        } else if (tid < 512) {     // gv
            if (ft < nt) {
                float4 a = *reinterpret_cast<const float4 *>(&s_pv[0][ft][fc]);
#pragma unroll
                for (int qq = 1; qq < NWR; ++qq) {
                    const float4 c = *reinterpret_cast<const float4 *>(&s_pv[qq][ft][fc]);
                    a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
                }
                const float4 g4 = *reinterpret_cast<const float4 *>(&s_g[ft][fc]);
                const float ruk = s_ruk[ft];
                store4(gv + of, fmaf(g4.x, ruk, a.x), fmaf(g4.y, ruk, a.y), fmaf(g4.z, ruk, a.z), fmaf(g4.w, ruk, a.w));
            }
        }
        __syncthreads();
        if (tid < 256) {
            // sum_{m>t} (P_m - Q_m) over the rows after mine in this tile, plus all later tiles
            float suf[4] = {carry[0], carry[1], carry[2], carry[3]};
            float tot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int m = TC - 1; m >= 0; --m) {
                const float4 e4 = *reinterpret_cast<const float4 *>(&s_e[m][fc]);
                if (m > ft) { suf[0] += e4.x; suf[1] += e4.y; suf[2] += e4.z; suf[3] += e4.w; }
                tot[0] += e4.x; tot[1] += e4.y; tot[2] += e4.z; tot[3] += e4.w;
            }
            if (ft < nt) {
                float o4[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // gw carries a factor d_t; once d_t underflows to 0 the value is 0, and without
                    // this guard exp(w_t) would amplify the rounding residue of the running sums
                    const float ew = fast_exp(curW[i]);
                    o4[i] = (fast_exp(-ew) == 0.f) ? 0.f : -ew * (suf[i] - Qv[i]);
                }
                // the first and last decay never reach an output: exactly zero, as the reference
                // kernel writes them (rwkv_kernels.cu:381,406), not the rounding residue of P - Q
                // (with a gradient arriving at the final state / a non-zero initial state they do)
                if ((t0 + ft == 0 && first_decay_unused) || (t0 + ft == T - 1 && !gsT)) { o4[0] = o4[1] = o4[2] = o4[3] = 0.f; }
                store4(gw + of, o4[0], o4[1], o4[2], o4[3]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) carry[i] += tot[i];
        }
        // s_e is next written two barriers from here; staging overwrites only tiles whose readers
        // are done (finalisers read s_r/s_k/s_g/s_vgy/s_ruk before the barrier above).
    }
    if (gs0 && role_k) {
#pragma unroll
        for (int i = 0; i < RW; ++i) gs0[lane * kN + RW * q + i] = g[i];
    }
}


}  // namespace wkv6
