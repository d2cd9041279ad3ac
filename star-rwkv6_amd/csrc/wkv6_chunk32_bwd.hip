// Backward of the full-precision chunk form (see wkv6_chunk32.h): fp32 and fp16 tensors, gradients fp32-exact
// to rounding, every product on v_mfma_f32_16x16x4_f32.
//
// Chunks of 32 tokens from the last to the first.  With S_0 the state at the chunk's start (saved by the
// forward), G = dL/dS at its end, B[t][s] = sum_j gy_t[j] v_s[j] (s < t), vgy_t = B[t][t], A as in the forward:
//   gv_s = K'_s G + sum_{t>=s} A[t][s] gy_t                       (A's diagonal holds sum_i r u k)
//   gr_t = e^{c_t} o Z_t + u k_t vgy_t ,    Z_t = gy_t S_0^T + e^{-m} o sum_{s<t} B[t][s] K~_s
//   gk_s = e^{c_32-c_{s+1}} o W_s + u r_s vgy_s ,  W_s = v_s G^T + e^{m-c_32} o sum_{t>s} B[t][s] R~_t
//   gu  += r_t k_t vgy_t
//   G   <- e^{c_32} o G + R'^T gy
//   gw_t = d_t (E_{t+1} - K'_t W_t) ,  E_t = E_{t+1} + R'_t Z_t - K'_t W_t ,  E_T = 0
// (E_t[i] = sum_j S_t[i][j] G_t[i][j]: what flows into channel i's decay at token t is the balance of what
// the later tokens read from the state and what they wrote to it.)
//
// One workgroup of twelve waves per (batch, head) pair, three roles of four waves (one wave of each role per SIMD,
// so that one role's waits are another's issue slots):
//   loading waves   tiles r, k, e^{c_t}, e^{c_32-c_{t+1}}, v, gy, d of the next chunk -> LDS (loads issued one phase
//                   ahead of their use: the kernel is bound by arithmetic, not by memory)
//   value waves     wave q owns value columns 16q.. of G: gv = K' G + A^T gy, the update of G, the tiles of A
//   key waves       wave q owns key rows 16q.. of G^T and of every per-channel output: Z, W, gr, gk, gw, gu, the
//                   update of G^T, the tiles of B; S_0^T comes straight from the saved states
// Both G and G^T are kept so that neither K' G nor v G^T needs a sum across waves.  Two workgroup barriers per chunk:
//   phase 1  tiles of A and B -> LDS ; K' G ; gy S_0^T ; v G^T
//   phase 2  the three products with A and B ; gradients out (16 lanes x 4 bytes per row piece) ; G, G^T updates
#include "wkv6_chunk32.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>

namespace wkv6 {

struct C32BwdLds {
    float R[2][kC32][kLd], K[2][kC32][kLd], F1[2][kC32][kLd], F3[2][kC32][kLd];   // r, k, e^{c_t}, e^{c_32 - c_{t+1}}
    float V[2][kC32][kLd], GY[2][kC32][kLd], D[2][kC32][kLd];                     // v, gy, log decay
    float A[kC32][kLa], Bm[kC32][kLa];
    float e_all[2][kN], e_mid[2][kN], e_rest[2][kN], inv0[2][kN], inv1[2][kN];    // e^{c_32}, e^{m}, e^{c_32-m}, e^{-m}, e^{m-c_32}
    float ruk[2][4][kC32];
    float vgy[kC32];
    int wild[4];
};
union C32BwdSmem {
    C32BwdLds chunk;
    ScanBwdALds scan_a;
    ScanBwdBLds scan_b;
};

struct C32BwdArgs {
    int T, H;
    const void *r, *k, *v, *w, *u, *gy;
    void *gr, *gk, *gv, *gw, *gu;
    float *saved;   // [pair][chunk][4096] chunk-start states as the forward leaves them (fragment order)
    // gradients through the state, [pair][key][value] fp32, all null for the stateless operator: the initial state
    // (only the per-timestep second pass reads it: the chunk states already contain it), the gradient arriving at
    // the final state, the final state itself (read where gsT is given: E_T = sum_j S_T o gsT), dL/dS_0 (out)
    const float *s0, *gsT, *sT;
    float *gs0;
};

template <typename Tin, typename Tout>
__global__ __launch_bounds__(768) void chunk32_bwd_kernel(const C32BwdArgs a)
{
    extern __shared__ __align__(16) unsigned char c32_smem[];
    C32BwdLds &L = reinterpret_cast<C32BwdSmem *>(c32_smem)->chunk;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int T = a.T, H = a.H;
    const int pair = blockIdx.x, b = pair / H, h = pair - b * H;
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
    const int nchunk = (T + kC32 - 1) / kC32;
    const Tin *r = reinterpret_cast<const Tin *>(a.r), *k = reinterpret_cast<const Tin *>(a.k);
    const Tin *v = reinterpret_cast<const Tin *>(a.v), *w = reinterpret_cast<const Tin *>(a.w);
    const Tin *u = reinterpret_cast<const Tin *>(a.u);
    const Tout *gy = reinterpret_cast<const Tout *>(a.gy);
    float *const ck = a.saved + (int64_t)pair * nchunk * (kN * kN);
    // step s handles chunk nchunk - 1 - s

    if (wave >= 8) {
        // ---------------- loading waves ----------------
        const int p = wave - 8, t16 = lane & 15, ch = 16 * p + 4 * (lane >> 4);
        float fu[4];
        load4(u + h * kN + ch, fu);
        float nr[2][4], nk[2][4], nv[2][4], nw[2][4], ng[2][4];   // the group's chunk as loaded (r, k, v, gy stay until handed on)
        auto fetch = [&](int s) {
            const int c = nchunk - 1 - s;
            const int64_t row0 = base + (int64_t)c * kC32 * C;   // (uniform)
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int o = min(16 * x + t16, T - 1 - c * kC32) * (int)C + ch;   // rows past the end read the last one
                load4(r + row0 + o, nr[x]); load4(k + row0 + o, nk[x]); load4(v + row0 + o, nv[x]); load4(w + row0 + o, nw[x]);
                load4(gy + row0 + o, ng[x]);
            }
        };
        float f1[2][4], f3[2][4], dd[2][4], e_all[4], e_mid[4], e_rest[4], inv0[4], inv1[4], part[2];
        bool wild = false;
        // two channels of the lane's four at a time (a barrier in between)
        auto form = [&](auto half, int s) {
            constexpr int E0 = 2 * decltype(half)::value;
            const int c = nchunk - 1 - s;
            const bool valid[2] = {c * kC32 + t16 < T, c * kC32 + 16 + t16 < T};
            C32Scale sc;
            sc.wild = false;
            c32_scale<E0, E0 + 2>(nw, valid, sc, dd);
            wild |= sc.wild;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                float acc = E0 == 0 ? 0.f : part[x];
#pragma unroll
                for (int e = E0; e < E0 + 2; ++e) {
                    if (!valid[x]) { nr[x][e] = 0.f; nk[x][e] = 0.f; nv[x][e] = 0.f; ng[x][e] = 0.f; }
                    f1[x][e] = sc.rp[x][e];
                    f3[x][e] = sc.kp[x][e];
                    e_all[e] = sc.all[e]; e_mid[e] = sc.mid[e]; e_rest[e] = sc.rest[e]; inv0[e] = sc.inv0[e]; inv1[e] = sc.inv1[e];
                    acc = fmaf(nr[x][e] * nk[x][e], fu[e], acc);
                }
                part[x] = E0 == 0 ? acc : sum_rows4(acc);
            }
        };
        auto as4 = [](const float (&f)[4]) { return (f32x4){f[0], f[1], f[2], f[3]}; };
        auto publish = [&](int s) {
            const int buf = s & 1;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int t = 16 * x + t16;
                *reinterpret_cast<f32x4 *>(&L.R[buf][t][ch]) = as4(nr[x]);
                *reinterpret_cast<f32x4 *>(&L.K[buf][t][ch]) = as4(nk[x]);
                *reinterpret_cast<f32x4 *>(&L.F1[buf][t][ch]) = as4(f1[x]);
                *reinterpret_cast<f32x4 *>(&L.F3[buf][t][ch]) = as4(f3[x]);
                *reinterpret_cast<f32x4 *>(&L.V[buf][t][ch]) = as4(nv[x]);
                *reinterpret_cast<f32x4 *>(&L.GY[buf][t][ch]) = as4(ng[x]);
                *reinterpret_cast<f32x4 *>(&L.D[buf][t][ch]) = as4(dd[x]);
                if (lane < 16) L.ruk[buf][p][t] = part[x];
            }
            if (t16 == 0) {
                *reinterpret_cast<f32x4 *>(&L.e_all[buf][ch]) = as4(e_all);
                *reinterpret_cast<f32x4 *>(&L.e_mid[buf][ch]) = as4(e_mid);
                *reinterpret_cast<f32x4 *>(&L.e_rest[buf][ch]) = as4(e_rest);
                *reinterpret_cast<f32x4 *>(&L.inv0[buf][ch]) = as4(inv0);
                *reinterpret_cast<f32x4 *>(&L.inv1[buf][ch]) = as4(inv1);
            }
        };
        const std::integral_constant<int, 0> h0;
        const std::integral_constant<int, 1> h1;
        // While step s is computed: the tiles of step s + 1 go to LDS and the loads of step s + 2 are issued
        // (phase 1), the scale factors of step s + 2 are formed (phase 2).
        fetch(0);
        form(h0, 0);
        form(h1, 0);
        publish(0);
        if (nchunk > 1) {
            fetch(1);
            form(h0, 1);
            form(h1, 1);
        }
        __syncthreads();
        for (int s = 0; s < nchunk; ++s) {
            if (s + 1 < nchunk) publish(s + 1);
            if (s + 2 < nchunk) fetch(s + 2);
            __syncthreads();
            if (s + 2 < nchunk) {
                form(h0, s + 2);
                form(h1, s + 2);
            }
            __syncthreads();
        }
        const bool any = __any(wild);
        if (lane == 0) L.wild[p] = any;
    } else if (wave < 4) {
        // ---------------- value waves ----------------
        const int q = wave, n = lane & 15, g = lane >> 4, col = 16 * q + n;
        Tout *gv = reinterpret_cast<Tout *>(a.gv);
        const f32x4 zero = (f32x4){0.f, 0.f, 0.f, 0.f};
        const int lane_off = 4 * g * (int)C + col;
        f32x4 G[4];   // G[ib][e] = G[16ib+4g+e][col]
#pragma unroll
        for (int i = 0; i < 4; ++i) G[i] = zero;
        if (a.gsT) {
            const float *p = a.gsT + (int64_t)pair * (kN * kN) + col;
#pragma unroll
            for (int ib = 0; ib < 4; ++ib)
#pragma unroll
                for (int e = 0; e < 4; ++e) G[ib][e] = p[(16 * ib + 4 * g + e) * kN];
        }
        __syncthreads();
        for (int s = 0; s < nchunk; ++s) {
            const int c = nchunk - 1 - s, buf = s & 1;
            const bool full = (c + 1) * kC32 <= T;
            // ---- phase 1: a tile of A (wave 0: (0,0), 1: (1,1), 2: (1,0)), K' G ----
            if (q < 3) {
                const int tb = q == 0 ? 0 : 1, sb = q == 1 ? 1 : 0;
                f32x4 at = zero;
#pragma unroll
                for (int ib = 0; ib < 4; ++ib) {
                    const int i0 = 16 * ib + 4 * g;
                    const f32x4 fk = *reinterpret_cast<const f32x4 *>(&L.K[buf][16 * sb + n][i0]) *
                                     *reinterpret_cast<const f32x4 *>(&L.F3[buf][16 * sb + n][i0]) *
                                     *reinterpret_cast<const f32x4 *>(&L.inv1[buf][i0]);
                    const f32x4 fr = *reinterpret_cast<const f32x4 *>(&L.R[buf][16 * tb + n][i0]) *
                                     *reinterpret_cast<const f32x4 *>(&L.F1[buf][16 * tb + n][i0]) *
                                     *reinterpret_cast<const f32x4 *>(&L.inv0[buf][i0]);
                    at = mfma16(fk, fr, at);
                }
                if (tb == sb) {
                    const int t = 16 * tb + n;
                    const float diag = (L.ruk[buf][0][t] + L.ruk[buf][1][t]) + (L.ruk[buf][2][t] + L.ruk[buf][3][t]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) at[e] = (4 * g + e < n) ? at[e] : (4 * g + e == n ? diag : 0.f);
                }
                *reinterpret_cast<f32x4 *>(&L.A[16 * tb + n][16 * sb + 4 * g]) = at;
            }
            f32x4 gvt[2] = {zero, zero};
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int ib = 0; ib < 4; ++ib) {
                    const f32x4 fk = *reinterpret_cast<const f32x4 *>(&L.K[buf][16 * sb + n][16 * ib + 4 * g]) *
                                     *reinterpret_cast<const f32x4 *>(&L.F3[buf][16 * sb + n][16 * ib + 4 * g]);
                    gvt[sb] = mfma16(fk, G[ib], gvt[sb]);
                }
            __syncthreads();
            // ---- phase 2: gv += A^T gy, out ; G <- e^{c_32} o G + R'^T gy ----
            f32x4 gyb[2];   // element e: token 16x + 4g + e, channel col
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int e = 0; e < 4; ++e) gyb[x][e] = L.GY[buf][16 * x + 4 * g + e][col];
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int tb = sb; tb < 2; ++tb) {
                    f32x4 fat;
#pragma unroll
                    for (int e = 0; e < 4; ++e) fat[e] = L.A[16 * tb + 4 * g + e][16 * sb + n];
                    gvt[sb] = mfma16(fat, gyb[tb], gvt[sb]);
                }
            {
                Tout *const out = gv + base + (int64_t)c * kC32 * C;   // (uniform; the lane's part of the address is lane_off)
                const int left = T - c * kC32 - 4 * g;                 // rows of the lane's four-row groups that exist
#pragma unroll
                for (int x = 0; x < 2; ++x)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (full || 16 * x + e < left) store1(out + (16 * x + e) * C + lane_off, gvt[x][e]);
            }
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) {
                G[ib] *= *reinterpret_cast<const f32x4 *>(&L.e_all[buf][16 * ib + 4 * g]);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    f32x4 fra;
#pragma unroll
                    for (int e = 0; e < 4; ++e) fra[e] = L.R[buf][16 * tb + 4 * g + e][16 * ib + n] * L.F1[buf][16 * tb + 4 * g + e][16 * ib + n];
                    G[ib] = mfma16(fra, gyb[tb], G[ib]);
                }
            }
            __syncthreads();
        }
        if (a.gs0) {   // what is left after the first chunk is dL/dS_0
            float *p = a.gs0 + (int64_t)pair * (kN * kN) + col;
#pragma unroll
            for (int ib = 0; ib < 4; ++ib)
#pragma unroll
                for (int e = 0; e < 4; ++e) p[(16 * ib + 4 * g + e) * kN] = G[ib][e];
        }
    } else {
        // ---------------- key waves ----------------
        const int q = wave - 4, n = lane & 15, g = lane >> 4, col = 16 * q + n;
        Tout *gr = reinterpret_cast<Tout *>(a.gr), *gk = reinterpret_cast<Tout *>(a.gk), *gw = reinterpret_cast<Tout *>(a.gw);
        const f32x4 zero = (f32x4){0.f, 0.f, 0.f, 0.f};
        const int lane_off = 4 * g * (int)C + col;
        f32x4 Gt[4], St[4];   // Gt[jb][e] = G[col][16jb+4g+e] ; St likewise of S_0
#pragma unroll
        for (int i = 0; i < 4; ++i) Gt[i] = zero;
        float E = 0.f, gu_acc = 0.f;
        if (a.gsT) {   // G_T^T, and the anchor of the decay gradient's sums: E_T = sum_j S_T o G_T over the row
            const float *pg = a.gsT + (int64_t)pair * (kN * kN) + col * kN + 4 * g;
            const float *ps = a.sT + (int64_t)pair * (kN * kN) + col * kN + 4 * g;
            float part = 0.f;
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                Gt[jb] = *reinterpret_cast<const f32x4 *>(pg + 16 * jb);
                const f32x4 sv = *reinterpret_cast<const f32x4 *>(ps + 16 * jb);
                part += (sv[0] * Gt[jb][0] + sv[1] * Gt[jb][1]) + (sv[2] * Gt[jb][2] + sv[3] * Gt[jb][3]);
            }
            E = sum_rows4(part);
        }
        const float u_lane = load1(u + h * kN + col);
        // S_0^T from the forward's fragment order: S[i][j] sits in tile (j / 16, i / 16) at lane (j % 16) + 16 ((i % 16) / 4), element i % 4
        auto load_state = [&](int c) {
            const float *p0 = ck + (int64_t)c * (kN * kN) + (q * 64 + 4 * g + 16 * (n >> 2)) * 4 + (n & 3);
#pragma unroll
            for (int jb = 0; jb < 4; ++jb)
#pragma unroll
                for (int e = 0; e < 4; ++e) St[jb][e] = p0[jb * 1024 + e * 4];
        };
        load_state(nchunk - 1);
        __syncthreads();
        for (int s = 0; s < nchunk; ++s) {
            const int c = nchunk - 1 - s, buf = s & 1;
            const bool full = (c + 1) * kC32 <= T;
            // ---- phase 1: a tile of B (wave 0: (0,0), 1: (1,1), 3: (1,0)), gy S_0^T, v G^T ----
            if (q != 2) {
                const int tb = q == 0 ? 0 : 1, sb = q == 1 ? 1 : 0;
                f32x4 bt = zero;
#pragma unroll
                for (int jb = 0; jb < 4; ++jb) {
                    const f32x4 fv = *reinterpret_cast<const f32x4 *>(&L.V[buf][16 * sb + n][16 * jb + 4 * g]);
                    const f32x4 fg = *reinterpret_cast<const f32x4 *>(&L.GY[buf][16 * tb + n][16 * jb + 4 * g]);
                    bt = mfma16(fv, fg, bt);
                }
                if (tb == sb) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (4 * g + e == n) L.vgy[16 * tb + n] = bt[e];
                        bt[e] = (4 * g + e < n) ? bt[e] : 0.f;
                    }
                }
                *reinterpret_cast<f32x4 *>(&L.Bm[16 * tb + n][16 * sb + 4 * g]) = bt;
            }
            f32x4 Z[2] = {zero, zero}, W[2] = {zero, zero};
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int jb = 0; jb < 4; ++jb) {
                    const f32x4 fg = *reinterpret_cast<const f32x4 *>(&L.GY[buf][16 * x + n][16 * jb + 4 * g]);
                    const f32x4 fv = *reinterpret_cast<const f32x4 *>(&L.V[buf][16 * x + n][16 * jb + 4 * g]);
                    Z[x] = mfma16(fg, St[jb], Z[x]);
                    W[x] = mfma16(fv, Gt[jb], W[x]);
                }
            const float e_all = L.e_all[buf][col], e_mid = L.e_mid[buf][col], e_rest = L.e_rest[buf][col];
            const float inv0 = L.inv0[buf][col], inv1 = L.inv1[buf][col];
            // the products with B come scaled from the middle of the chunk: bring these to that scale, all back at the end
#pragma unroll
            for (int x = 0; x < 2; ++x) { Z[x] *= e_mid; W[x] *= e_rest; }
            if (c > 0) load_state(c - 1);
            __syncthreads();
            // ---- phase 2 ----
            f32x4 rc[2], kc[2], rp[2], kp[2];   // element e: token 16x + 4g + e, channel col
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int t = 16 * x + 4 * g + e;
                    rc[x][e] = L.R[buf][t][col];
                    kc[x][e] = L.K[buf][t][col];
                    rp[x][e] = rc[x][e] * L.F1[buf][t][col];
                    kp[x][e] = kc[x][e] * L.F3[buf][t][col];
                }
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int sb = 0; sb <= tb; ++sb) {
                    const f32x4 fb = *reinterpret_cast<const f32x4 *>(&L.Bm[16 * tb + n][16 * sb + 4 * g]);
                    Z[tb] = mfma16(fb, kp[sb] * inv1, Z[tb]);
                }
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int tb = sb; tb < 2; ++tb) {
                    f32x4 fbt;
#pragma unroll
                    for (int e = 0; e < 4; ++e) fbt[e] = L.Bm[16 * tb + 4 * g + e][16 * sb + n];
                    W[sb] = mfma16(fbt, rp[tb] * inv0, W[sb]);
                }
            // G^T <- e^{c_32} o G^T + gy^T R' (before the outputs: they need no matrix unit)
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                Gt[jb] *= e_all;
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    f32x4 fga;
#pragma unroll
                    for (int e = 0; e < 4; ++e) fga[e] = L.GY[buf][16 * tb + 4 * g + e][16 * jb + n];
                    Gt[jb] = mfma16(fga, rp[tb], Gt[jb]);
                }
            }
            // gradients out
            float zt[2][4], kgk[2][4];
            const int64_t out0 = base + (int64_t)c * kC32 * C;   // (uniform; the lane's part of the address is lane_off)
            const int left = T - c * kC32 - 4 * g;               // rows of the lane's four-row groups that exist
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const f32x4 vg = *reinterpret_cast<const f32x4 *>(&L.vgy[16 * x + 4 * g]);
                Z[x] *= inv0;
                W[x] *= inv1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int tl = 16 * x + 4 * g + e;
                    const float f1 = L.F1[buf][tl][col], f3 = L.F3[buf][tl][col];
                    const float o_r = fmaf(f1, Z[x][e], u_lane * kc[x][e] * vg[e]);
                    const float o_k = fmaf(f3, W[x][e], u_lane * rc[x][e] * vg[e]);
                    kgk[x][e] = kp[x][e] * W[x][e];
                    zt[x][e] = fmaf(rp[x][e], Z[x][e], -kgk[x][e]);
                    gu_acc = fmaf(rc[x][e] * kc[x][e], vg[e], gu_acc);
                    if (full || 16 * x + e < left) {
                        store1(gr + out0 + (16 * x + e) * C + lane_off, o_r);
                        store1(gk + out0 + (16 * x + e) * C + lane_off, o_k);
                    }
                }
            }
            {   // E_{t+1} = E at the chunk's end + what the later tokens of the chunk add
                float tot[2], other[2][4], later[2];
#pragma unroll
                for (int x = 0; x < 2; ++x) {
                    tot[x] = (zt[x][0] + zt[x][1]) + (zt[x][2] + zt[x][3]);
                    rows4(tot[x], other[x]);
                    later[x] = (g < 1 ? other[x][1] : 0.f) + (g < 2 ? other[x][2] : 0.f) + (g < 3 ? other[x][3] : 0.f);
                }
                const float all1 = (other[1][0] + other[1][1]) + (other[1][2] + other[1][3]);
                const float all0 = (other[0][0] + other[0][1]) + (other[0][2] + other[0][3]);
                later[0] += all1;
#pragma unroll
                for (int x = 0; x < 2; ++x) {
                    float run = E + later[x];
#pragma unroll
                    for (int e = 3; e >= 0; --e) {
                        const int tl = 16 * x + 4 * g + e;
                        float o_w = (run - kgk[x][e]) * L.D[buf][tl][col];
                        // (a zero initial state: the first decay reaches no output, its gradient is zero and not
                        // what rounding leaves of two equal sums)
                        if (x == 0 && e == 0 && a.s0 == nullptr && c == 0 && g == 0) o_w = 0.f;
                        if (full || 16 * x + e < left) store1(gw + out0 + (16 * x + e) * C + lane_off, o_w);
                        run += zt[x][e];
                    }
                }
                E += all0 + all1;
            }
            __syncthreads();
        }
        // gu: the four row groups of the wave hold the tokens 4g .. 4g+3 (mod 16) of every chunk
        gu_acc = sum_rows4(gu_acc);
        if (g == 0) store1(reinterpret_cast<Tout *>(a.gu) + (int64_t)b * C + h * kN + col, gu_acc);
    }
    __syncthreads();
    // a pair whose decay left the reach: once more, one timestep at a time (the pair's slice of the saved
    // states, T/32 x 64 x 64 floats, is large enough for the T x 64 workspace of that pass)
    __shared__ float s_ft[kN];
    if (L.wild[0] | L.wild[1] | L.wild[2] | L.wild[3]) {
        const int64_t so = (int64_t)pair * (kN * kN);
        const float *s0p = a.s0 ? a.s0 + so : nullptr, *gsTp = a.gsT ? a.gsT + so : nullptr;
        float *gs0p = a.gs0 ? a.gs0 + so : nullptr;
        const bool states = s0p || gsTp || gs0p;
        __syncthreads();
        scan_bwd_a_body<Tin, Tout>(reinterpret_cast<C32BwdSmem *>(c32_smem)->scan_a, b, h, T, H, r, k, v, w, u, gy,
                                   reinterpret_cast<Tout *>(a.gr), reinterpret_cast<Tout *>(a.gu), ck, kN,
                                   s0p, gsTp, states ? s_ft : nullptr);
        __threadfence_block();
        __syncthreads();
        scan_bwd_b_body<Tin, Tout>(reinterpret_cast<C32BwdSmem *>(c32_smem)->scan_b, b, h, T, H, r, k, v, w, u, gy, ck, kN,
                                   reinterpret_cast<Tout *>(a.gk), reinterpret_cast<Tout *>(a.gv), reinterpret_cast<Tout *>(a.gw),
                                   gsTp, states ? s_ft : nullptr, gs0p, s0p == nullptr);
    }
}

template <typename Tin, typename Tout>
static hipError_t launch(hipStream_t st, int64_t B, const C32BwdArgs &a) {
    constexpr int lds = (int)sizeof(C32BwdSmem);
    const hipError_t e = allow_dynamic_lds<chunk32_bwd_kernel<Tin, Tout>>(lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((chunk32_bwd_kernel<Tin, Tout>), dim3((unsigned)(B * a.H)), dim3(768), lds, st, a);
    return hipGetLastError();
}

hipError_t chunk32_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                            const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                            void *gr, void *gk, void *gv, void *gw, void *gu, void *saved_states,
                            const float *s0, const float *gsT, const float *sT, float *gs0)
{
    if (gsT != nullptr && sT == nullptr) return hipErrorInvalidValue;   // (the anchor of the decay gradient needs S_T)
    C32BwdArgs a;
    a.s0 = s0; a.gsT = gsT; a.sT = sT; a.gs0 = gs0;
    a.T = (int)T; a.H = (int)H;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu;
    a.saved = reinterpret_cast<float *>(saved_states);
    if (dtype == kF32) return launch<float, float>(st, B, a);
    return launch<f16_t, float>(st, B, a);
}

}  // namespace wkv6
