// WKV6 for head sizes other than 64 (any multiple of 4 up to 128): the per-timestep recurrence in fp32, one
// thread per channel.  The reference builds its kernels for any head size that is a multiple of 4
// (rwkv_kernel/torch_rwkv_kernel.py:13, rwkv_kernel/jax_kernel/rwkv_kernels.cu:101) and its own scripts run 8
// and 32; the models all use 64, which has the tuned kernels of this library.  This file serves the rest of
// the interface, not a benchmark.
//
// The kernels are built for head sizes up to kMax = 8, 16, 32, 64, 128 and take the head size N <= kMax at run
// time (the loops over a head's channels are unrolled to kMax and guarded, so the state stays in registers).
// A workgroup of kW = max(64, kMax) threads takes the kW / N whole heads that fit (their channels are
// consecutive) of one batch row; threads beyond them idle.  Tiles of 16 timesteps of the inputs are staged
// through LDS as fp32; the values of a thread's head that are the same for all of its threads (r, k, u, the
// decay, or v, gy) are broadcast reads.
//   forward   thread (h, j) owns column j of the head's state
//   sweep A   (time ascending)  thread (h, i) owns row i of the state: gr, gu, P_t = r_t (gr_t without the u term)
//   sweep B   (time descending) the reverse state twice, row i and column j: gk, gv, and gw through
//             gw_t = d_t (E_{t+1} - k_t gk'_t), E_t = E_{t+1} + P_t - k_t gk'_t  (gk' = gk without the u term)
// Gradients through the state: S_0 = s0, G_T = gsT, E_T = sum_j S_T o G_T (left by sweep A), gs0 = G_0.
#include "wkv6_common.h"
#include "wkv6_kernels.h"

namespace wkv6 {

constexpr int kGenTile = 16;   // timesteps per LDS tile
constexpr int gen_width(int kMax) { return kMax > 64 ? kMax : 64; }   // threads of a workgroup

struct GenArgs {
    int T, H, N;
    const void *r, *k, *v, *w, *u, *gy;
    const void *s0;              // forward: (rows, H, N, N) in the state type; backward: (B, H, N, N) fp32
    const int64_t *map;
    void *y, *sT;
    void *gr, *gk, *gv, *gw, *gu;
    float *wsP;                  // (B, T, C) fp32, then (B, C) for E_T
    const float *gsT;
    float *gs0;
};

// what a thread works on: channel c = head h, position i inside the head; hb = the head's first thread
struct GenLane {
    bool live;
    int c, h, i, hb;
    int64_t first;               // (b, 0, c) in a (B, T, C) tensor
};
template <int kW>
__device__ __forceinline__ GenLane gen_lane(const GenArgs &a) {
    const int N = a.N, heads = kW / N, tid = threadIdx.x;
    const int64_t C = (int64_t)a.H * N;
    GenLane l;
    const bool used = tid < heads * N;   // the threads behind the last whole head idle (and read head 0's LDS columns)
    l.i = tid % N;
    l.hb = used ? tid - l.i : 0;
    const int64_t c = (int64_t)blockIdx.x * heads * N + tid;
    l.live = used && c < C;
    l.c = l.live ? (int)c : 0;
    l.h = l.c / N;
    l.first = (int64_t)blockIdx.y * a.T * C + l.c;
    return l;
}

// one tile of a (B, T, C) tensor -> LDS (the thread's own channel; rows past the end: `fill`)
template <int kW, typename T>
__device__ __forceinline__ void gen_stage(float (&dst)[kGenTile][kW], const T *src, int64_t first, int64_t C, int t0, int Tn, bool live, float fill) {
#pragma unroll
    for (int t = 0; t < kGenTile; ++t)
        dst[t][threadIdx.x] = (live && t0 + t < Tn) ? load1(src + first + (int64_t)(t0 + t) * C) : fill;
}
template <int kW, typename T>
__device__ __forceinline__ void gen_stage_decay(float (&dst)[kGenTile][kW], const T *w, int64_t first, int64_t C, int t0, int Tn, bool live) {
#pragma unroll
    for (int t = 0; t < kGenTile; ++t)
        dst[t][threadIdx.x] = (live && t0 + t < Tn) ? decay_from_raw(load1(w + first + (int64_t)(t0 + t) * C)) : 1.f;
}

template <int kMax, typename Tin, typename Tout, typename Ts>
__global__ __launch_bounds__(gen_width(kMax)) void gen_fwd_kernel(const GenArgs a)
{
    constexpr int kW = gen_width(kMax);
    __shared__ float s_r[kGenTile][kW], s_k[kGenTile][kW], s_d[kGenTile][kW], s_v[kGenTile][kW], s_u[kW];
    const int T = a.T, H = a.H, N = a.N, b = blockIdx.y, tid = threadIdx.x;
    const int64_t C = (int64_t)H * N;
    const GenLane l = gen_lane<kW>(a);
    const bool live = l.live;
    const int j = l.i, hb = l.hb;
    const int64_t first = l.first;
    const Tin *r = (const Tin *)a.r, *k = (const Tin *)a.k, *v = (const Tin *)a.v, *w = (const Tin *)a.w, *u = (const Tin *)a.u;
    s_u[tid] = live ? load1(u + l.c) : 0.f;
    float S[kMax];   // column j of the state
#pragma unroll
    for (int i = 0; i < kMax; ++i) S[i] = 0.f;
    if (a.s0 && live) {
        const int64_t row = a.map ? a.map[b] : (int64_t)b;
        const Ts *p = (const Ts *)a.s0 + ((row * H + l.h) * N) * N + j;
#pragma unroll
        for (int i = 0; i < kMax; ++i)
            if (i < N) S[i] = load1(p + i * N);
    }
    for (int t0 = 0; t0 < T; t0 += kGenTile) {
        __syncthreads();
        gen_stage<kW>(s_r, r, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_k, k, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_v, v, first, C, t0, T, live, 0.f);
        gen_stage_decay<kW>(s_d, w, first, C, t0, T, live);
        __syncthreads();
        const int nt = min(kGenTile, T - t0);
        for (int t = 0; t < nt; ++t) {
            const float vj = s_v[t][tid];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < kMax; ++i)
                if (i < N) {
                    const float ri = s_r[t][hb + i], ki = s_k[t][hb + i], di = s_d[t][hb + i];
                    const float x = ki * vj;
                    acc = fmaf(ri, fmaf(s_u[hb + i], x, S[i]), acc);
                    S[i] = fmaf(S[i], di, x);
                }
            if (live && a.y) store1((Tout *)a.y + first + (int64_t)(t0 + t) * C, acc);
        }
    }
    if (a.sT && live) {
        Ts *p = (Ts *)a.sT + (((int64_t)b * H + l.h) * N) * N + j;
#pragma unroll
        for (int i = 0; i < kMax; ++i)
            if (i < N) store1(p + i * N, S[i]);
    }
}

template <int kMax, typename Tin, typename Tout>
__global__ __launch_bounds__(gen_width(kMax)) void gen_bwd_a_kernel(const GenArgs a)
{
    constexpr int kW = gen_width(kMax);
    __shared__ float s_v[kGenTile][kW], s_g[kGenTile][kW];
    const int T = a.T, H = a.H, N = a.N, b = blockIdx.y;
    const int64_t C = (int64_t)H * N;
    const GenLane l = gen_lane<kW>(a);
    const bool live = l.live;
    const int i = l.i, hb = l.hb, c = l.c;
    const int64_t first = l.first;
    const Tin *r = (const Tin *)a.r, *k = (const Tin *)a.k, *v = (const Tin *)a.v, *w = (const Tin *)a.w;
    const Tout *gy = (const Tout *)a.gy;
    const float ui = live ? load1((const Tin *)a.u + c) : 0.f;
    float S[kMax];   // row i of the state
#pragma unroll
    for (int jj = 0; jj < kMax; ++jj) S[jj] = 0.f;
    if (a.s0 && live) {
        const float *p = (const float *)a.s0 + (((int64_t)b * H + l.h) * N + i) * N;
#pragma unroll
        for (int jj = 0; jj < kMax; ++jj)
            if (jj < N) S[jj] = p[jj];
    }
    float gu = 0.f;
    for (int t0 = 0; t0 < T; t0 += kGenTile) {
        __syncthreads();
        gen_stage<kW>(s_v, v, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_g, gy, first, C, t0, T, live, 0.f);
        __syncthreads();
        const int nt = min(kGenTile, T - t0);
        for (int t = 0; t < nt; ++t) {
            const int64_t o = first + (int64_t)(t0 + t) * C;
            const float ri = live ? load1(r + o) : 0.f, ki = live ? load1(k + o) : 0.f;
            const float di = live ? decay_from_raw(load1(w + o)) : 1.f;
            float x = 0.f, vgy = 0.f;
#pragma unroll
            for (int jj = 0; jj < kMax; ++jj)
                if (jj < N) {
                    const float vj = s_v[t][hb + jj], gj = s_g[t][hb + jj];
                    x = fmaf(gj, S[jj], x);
                    vgy = fmaf(vj, gj, vgy);
                    S[jj] = fmaf(S[jj], di, ki * vj);
                }
            if (live) {
                store1((Tout *)a.gr + o, fmaf(ui * ki, vgy, x));
                a.wsP[o] = ri * x;
            }
            gu = fmaf(ri * ki, vgy, gu);
        }
    }
    if (live) {
        store1((Tout *)a.gu + (int64_t)b * C + c, gu);
        if (a.gsT) {   // E_T[i] = sum_j S_T[i][j] G_T[i][j]
            const float *p = a.gsT + (((int64_t)b * H + l.h) * N + i) * N;
            float e = 0.f;
#pragma unroll
            for (int jj = 0; jj < kMax; ++jj)
                if (jj < N) e = fmaf(S[jj], p[jj], e);
            a.wsP[(int64_t)gridDim.y * T * C + (int64_t)b * C + c] = e;
        }
    }
}

template <int kMax, typename Tin, typename Tout>
__global__ __launch_bounds__(gen_width(kMax)) void gen_bwd_b_kernel(const GenArgs a)
{
    constexpr int kW = gen_width(kMax);
    __shared__ float s_r[kGenTile][kW], s_k[kGenTile][kW], s_d[kGenTile][kW], s_v[kGenTile][kW], s_g[kGenTile][kW], s_u[kW];
    const int T = a.T, H = a.H, N = a.N, b = blockIdx.y, tid = threadIdx.x;
    const int64_t C = (int64_t)H * N;
    const GenLane l = gen_lane<kW>(a);
    const bool live = l.live;
    const int i = l.i, hb = l.hb, c = l.c;
    const int64_t first = l.first;
    const Tin *r = (const Tin *)a.r, *k = (const Tin *)a.k, *v = (const Tin *)a.v, *w = (const Tin *)a.w, *u = (const Tin *)a.u;
    const Tout *gy = (const Tout *)a.gy;
    const float ui = live ? load1(u + c) : 0.f;
    s_u[tid] = ui;
    float Gr[kMax], Gc[kMax];   // row i and column i of the reverse state
#pragma unroll
    for (int x = 0; x < kMax; ++x) { Gr[x] = 0.f; Gc[x] = 0.f; }
    float E = 0.f;
    if (a.gsT && live) {
        const float *p = a.gsT + ((int64_t)b * H + l.h) * N * N;
#pragma unroll
        for (int x = 0; x < kMax; ++x)
            if (x < N) { Gr[x] = p[i * N + x]; Gc[x] = p[x * N + i]; }
        E = a.wsP[(int64_t)gridDim.y * T * C + (int64_t)b * C + c];
    }
    const int ntile = (T + kGenTile - 1) / kGenTile;
    for (int tile = ntile - 1; tile >= 0; --tile) {
        const int t0 = tile * kGenTile;
        __syncthreads();
        gen_stage<kW>(s_r, r, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_k, k, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_v, v, first, C, t0, T, live, 0.f);
        gen_stage<kW>(s_g, gy, first, C, t0, T, live, 0.f);
        gen_stage_decay<kW>(s_d, w, first, C, t0, T, live);
        __syncthreads();
        const int nt = min(kGenTile, T - t0);
        for (int t = nt - 1; t >= 0; --t) {
            const int64_t o = first + (int64_t)(t0 + t) * C;
            const float ri = s_r[t][tid], ki = s_k[t][tid], di = s_d[t][tid], gi = s_g[t][tid];
            float vgy = 0.f, ruk = 0.f, q = 0.f, gvv = 0.f;
#pragma unroll
            for (int x = 0; x < kMax; ++x)
                if (x < N) {
                    const float rx = s_r[t][hb + x], kx = s_k[t][hb + x], dx = s_d[t][hb + x], vx = s_v[t][hb + x], gx = s_g[t][hb + x];
                    vgy = fmaf(vx, gx, vgy);
                    ruk = fmaf(rx * kx, s_u[hb + x], ruk);
                    q = fmaf(vx, Gr[x], q);
                    gvv = fmaf(kx, Gc[x], gvv);
                    Gr[x] = fmaf(Gr[x], di, ri * gx);
                    Gc[x] = fmaf(Gc[x], dx, rx * gi);
                }
            if (live) {
                const float logd = -fast_exp(load1(w + o));
                const bool ends = (t0 + t == 0 && a.s0 == nullptr);   // the first decay multiplies a zero state: no gradient
                store1((Tout *)a.gk + o, fmaf(ui * ri, vgy, q));
                store1((Tout *)a.gv + o, fmaf(ruk, gi, gvv));
                store1((Tout *)a.gw + o, ends ? 0.f : logd * (E - ki * q));
                E += a.wsP[o] - ki * q;
            }
        }
    }
    if (a.gs0 && live) {
        float *p = a.gs0 + (((int64_t)b * H + l.h) * N + i) * N;
#pragma unroll
        for (int x = 0; x < kMax; ++x)
            if (x < N) p[x] = Gr[x];
    }
}

// 64 has kernels of its own; everything else that the reference accepts (a multiple of 4) up to 128
bool generic_head_size(int64_t N) { return N >= 4 && N <= 128 && N % 4 == 0 && N != 64; }

static dim3 gen_grid(int kW, int64_t B, const GenArgs &a) {
    const int heads = kW / a.N;   // whole heads per workgroup
    return dim3((unsigned)((a.H + heads - 1) / heads), (unsigned)B);
}
template <int kMax, typename Tin, typename Tout, typename Ts>
static hipError_t gen_fwd_launch(hipStream_t st, int64_t B, const GenArgs &a) {
    constexpr int kW = gen_width(kMax);
    hipLaunchKernelGGL((gen_fwd_kernel<kMax, Tin, Tout, Ts>), gen_grid(kW, B, a), dim3(kW), 0, st, a);
    return hipGetLastError();
}
template <int kMax, typename Tin, typename Tout>
static hipError_t gen_bwd_launch(hipStream_t st, int64_t B, const GenArgs &a) {
    constexpr int kW = gen_width(kMax);
    hipLaunchKernelGGL((gen_bwd_a_kernel<kMax, Tin, Tout>), gen_grid(kW, B, a), dim3(kW), 0, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gen_bwd_b_kernel<kMax, Tin, Tout>), gen_grid(kW, B, a), dim3(kW), 0, st, a);
    return hipGetLastError();
}
template <int kMax>
static hipError_t gen_fwd_dtype(hipStream_t st, int dtype, int state_dtype, int64_t B, const GenArgs &a) {
    switch (dtype) {
    case kF32: return gen_fwd_launch<kMax, float, float, float>(st, B, a);
    case kF16: return gen_fwd_launch<kMax, f16_t, float, float>(st, B, a);
    default:   return state_dtype == kF32 ? gen_fwd_launch<kMax, bf16_t, bf16_t, float>(st, B, a) : gen_fwd_launch<kMax, bf16_t, bf16_t, bf16_t>(st, B, a);
    }
}
template <int kMax>
static hipError_t gen_bwd_dtype(hipStream_t st, int dtype, int64_t B, const GenArgs &a) {
    switch (dtype) {
    case kF32: return gen_bwd_launch<kMax, float, float>(st, B, a);
    case kF16: return gen_bwd_launch<kMax, f16_t, float>(st, B, a);
    default:   return gen_bwd_launch<kMax, bf16_t, bf16_t>(st, B, a);
    }
}

hipError_t generic_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                           const void *r, const void *k, const void *v, const void *w, const void *u,
                           const void *s0, const int64_t *map, void *y, void *sT)
{
    if (!generic_head_size(N) || B > 65535) return hipErrorInvalidValue;   // (the batch is the grid's second dimension)
    GenArgs a = {};
    a.T = (int)T; a.H = (int)H; a.N = (int)N;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.map = map; a.y = y; a.sT = sT;
    if (N <= 8)  return gen_fwd_dtype<8>(st, dtype, state_dtype, B, a);
    if (N <= 16) return gen_fwd_dtype<16>(st, dtype, state_dtype, B, a);
    if (N <= 32) return gen_fwd_dtype<32>(st, dtype, state_dtype, B, a);
    if (N <= 64) return gen_fwd_dtype<64>(st, dtype, state_dtype, B, a);
    return gen_fwd_dtype<128>(st, dtype, state_dtype, B, a);
}

size_t generic_backward_workspace_bytes(int64_t B, int64_t T, int64_t C) { return (size_t)(B * T * C + B * C) * sizeof(float); }

hipError_t generic_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const float *s0, const void *gy, const float *gsT,
                            void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0, void *workspace)
{
    if (!generic_head_size(N) || B > 65535) return hipErrorInvalidValue;
    GenArgs a = {};
    a.T = (int)T; a.H = (int)H; a.N = (int)N;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.gy = gy; a.s0 = s0; a.gsT = gsT; a.gs0 = gs0;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.wsP = (float *)workspace;
    if (N <= 8)  return gen_bwd_dtype<8>(st, dtype, B, a);
    if (N <= 16) return gen_bwd_dtype<16>(st, dtype, B, a);
    if (N <= 32) return gen_bwd_dtype<32>(st, dtype, B, a);
    if (N <= 64) return gen_bwd_dtype<64>(st, dtype, B, a);
    return gen_bwd_dtype<128>(st, dtype, B, a);
}

}  // namespace wkv6
