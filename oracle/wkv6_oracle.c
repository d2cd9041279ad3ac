/*
 * CPU restatement of the WKV6 time-mixing operator.  TEST INFRASTRUCTURE ONLY:
 * this file is the checker the HIP kernels are compared with; nothing that ships
 * (the rwkv_kernel package, the C-ABI library) may call it.
 *
 * Semantics followed (paths relative to the reference tree):
 *   forward  : rwkv_kernel/ops_rwkv_kernal.py:80-93  (python loop: kv_t = k_t (x) v_t,
 *              y_t = r_t @ (u*kv_t + s), s = kv_t + exp(-exp(w_t)) * s), which is the same
 *              arithmetic as rwkv_kernel/jax_kernel/rwkv_kernels.cu:122-159.
 *   state    : rwkv_kernel/ops_rwkv_kernal.py:41-72  (s = take(init_state, state_map, 0);
 *              state indexed [b][h][key j][value i]).
 *   backward : the gradients rwkv_kernel/jax_kernel/rwkv_kernels.cu:205-407 define
 *              (gr :242, gk :288, gv :333, per-batch gu :243-249, gw wrt the RAW w :404).
 *              They are evaluated here in the textbook adjoint form
 *                 G_t = r_t (x) gy_t + d_t * G_{t+1},   gw_t[j] = -exp(w_t[j]) d_t[j] sum_i S_t[j][i] G_{t+1}[j][i]
 *              with every forward state S_t kept in memory, i.e. NOT through the running-sum
 *              identity the reference kernel (and the HIP kernels) use for gw, so that the two
 *              derivations check each other.
 *
 * Built twice: REAL=double (arbiter) and REAL=float (fp32 arithmetic like the reference kernels).
 * Layout: r,k,v,w,y,gy,g* : (B,T,C) row-major, c = h*N + n;  u : (H,N);  state : (B,H,N,N) [key][value].
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL double
#endif
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

static inline REAL decay_of(REAL w) { return (REAL)exp(-exp((double)w)); }

/* Forward.  s0 may be NULL (zero state); if s0 is given, map (length B) selects the state row
 * (map may be NULL = identity).  sT may be NULL.  Returns 0, or -1 on a bad map entry. */
int FN(wkv6_oracle_forward)(int64_t B, int64_t T, int64_t H, int64_t N,
                            const REAL *r, const REAL *k, const REAL *v, const REAL *w, const REAL *u,
                            const REAL *s0, const int64_t *map, int64_t n_state,
                            REAL *y, REAL *sT)
{
    const int64_t C = H * N;
    int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad)
    for (int64_t bh = 0; bh < B * H; ++bh) {
        const int64_t b = bh / H, h = bh % H;
        REAL *S = (REAL *)calloc((size_t)(N * N), sizeof(REAL));
        if (s0) {
            int64_t row = map ? map[b] : b;
            if (row < 0 || row >= n_state) { bad |= 1; free(S); continue; }
            memcpy(S, s0 + (row * H + h) * N * N, (size_t)(N * N) * sizeof(REAL));
        }
        const REAL *uh = u + h * N;
        for (int64_t t = 0; t < T; ++t) {
            const int64_t o = (b * T + t) * C + h * N;
            for (int64_t i = 0; i < N; ++i) y[o + i] = 0;
            for (int64_t j = 0; j < N; ++j) {
                const REAL rj = r[o + j], kj = k[o + j], dj = decay_of(w[o + j]), uj = uh[j];
                REAL *Sj = S + j * N;
                for (int64_t i = 0; i < N; ++i) {
                    const REAL x = kj * v[o + i];
                    y[o + i] += rj * (uj * x + Sj[i]);
                    Sj[i] = x + dj * Sj[i];
                }
            }
        }
        if (sT) memcpy(sT + (b * H + h) * N * N, S, (size_t)(N * N) * sizeof(REAL));
        free(S);
    }
    return bad ? -1 : 0;
}

/* Backward.  S_0 = s0[b] (or 0 when s0 is NULL), G_T = gsT[b] (or 0): with both NULL this is the
 * backward of the stateless forward the reference defines (no gradient into or out of the state);
 * with states it is the gradient of  sum(y*gy) + sum(S_T*gsT)  and gs0 (if not NULL) receives
 * dL/dS_0 = G_0.  States are (B,H,N,N) in [key][value] order.
 * gu is written as per-batch partials (B,C), as the reference kernels do
 * (rwkv_kernels.cu:249); the batch sum is the caller's. */
static int backward_impl(int64_t B, int64_t T, int64_t H, int64_t N,
                         const REAL *r, const REAL *k, const REAL *v, const REAL *w, const REAL *u,
                         const REAL *s0, const REAL *gy, const REAL *gsT,
                         REAL *gr, REAL *gk, REAL *gv, REAL *gw, REAL *gu, REAL *gs0)
{
    const int64_t C = H * N, NN = N * N;
    int bad = 0;
#pragma omp parallel for schedule(dynamic) reduction(| : bad)
    for (int64_t bh = 0; bh < B * H; ++bh) {
        const int64_t b = bh / H, h = bh % H;
        REAL *Sall = (REAL *)malloc((size_t)(T * NN) * sizeof(REAL)); /* S_t before step t */
        REAL *G = (REAL *)calloc((size_t)NN, sizeof(REAL));
        if (!Sall || !G) { bad |= 1; free(Sall); free(G); continue; }
        const REAL *uh = u + h * N;
        /* forward sweep, keeping every state */
        if (s0) memcpy(Sall, s0 + bh * NN, (size_t)NN * sizeof(REAL));
        else memset(Sall, 0, (size_t)NN * sizeof(REAL));
        if (gsT) memcpy(G, gsT + bh * NN, (size_t)NN * sizeof(REAL));
        for (int64_t t = 0; t + 1 < T; ++t) {
            const int64_t o = (b * T + t) * C + h * N;
            const REAL *S = Sall + t * NN;
            REAL *Sn = Sall + (t + 1) * NN;
            for (int64_t j = 0; j < N; ++j) {
                const REAL kj = k[o + j], dj = decay_of(w[o + j]);
                for (int64_t i = 0; i < N; ++i) Sn[j * N + i] = kj * v[o + i] + dj * S[j * N + i];
            }
        }
        for (int64_t j = 0; j < N; ++j) gu[b * C + h * N + j] = 0;
        /* reverse sweep; G holds G_{t+1} on entry to step t */
        for (int64_t t = T - 1; t >= 0; --t) {
            const int64_t o = (b * T + t) * C + h * N;
            const REAL *S = Sall + t * NN;
            REAL vgy = 0;
            for (int64_t i = 0; i < N; ++i) { vgy += v[o + i] * gy[o + i]; gv[o + i] = 0; }
            for (int64_t j = 0; j < N; ++j) {
                const REAL rj = r[o + j], kj = k[o + j], uj = uh[j];
                const REAL ew = (REAL)exp((double)w[o + j]), dj = (REAL)exp(-(double)ew);
                REAL *Gj = G + j * N;
                REAL a_gr = 0, a_gk = 0, a_sg = 0;
                for (int64_t i = 0; i < N; ++i) {
                    const REAL gyi = gy[o + i], vi = v[o + i];
                    a_gr += gyi * (uj * kj * vi + S[j * N + i]);
                    a_gk += vi * (uj * rj * gyi + Gj[i]);
                    gv[o + i] += kj * (uj * rj * gyi + Gj[i]);
                    a_sg += S[j * N + i] * Gj[i];
                    Gj[i] = rj * gyi + dj * Gj[i];
                }
                gr[o + j] = a_gr;
                gk[o + j] = a_gk;
                gw[o + j] = -ew * dj * a_sg;
                gu[b * C + h * N + j] += rj * kj * vgy;
            }
        }
        if (gs0) memcpy(gs0 + bh * NN, G, (size_t)NN * sizeof(REAL));
        free(Sall);
        free(G);
    }
    return bad ? -1 : 0;
}

int FN(wkv6_oracle_backward)(int64_t B, int64_t T, int64_t H, int64_t N,
                             const REAL *r, const REAL *k, const REAL *v, const REAL *w, const REAL *u,
                             const REAL *gy,
                             REAL *gr, REAL *gk, REAL *gv, REAL *gw, REAL *gu)
{
    return backward_impl(B, T, H, N, r, k, v, w, u, NULL, gy, NULL, gr, gk, gv, gw, gu, NULL);
}

int FN(wkv6_oracle_backward_state)(int64_t B, int64_t T, int64_t H, int64_t N,
                                   const REAL *r, const REAL *k, const REAL *v, const REAL *w, const REAL *u,
                                   const REAL *s0, const REAL *gy, const REAL *gsT,
                                   REAL *gr, REAL *gk, REAL *gv, REAL *gw, REAL *gu, REAL *gs0)
{
    return backward_impl(B, T, H, N, r, k, v, w, u, s0, gy, gsT, gr, gk, gv, gw, gu, gs0);
}
