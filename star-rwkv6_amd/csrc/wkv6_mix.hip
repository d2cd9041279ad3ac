// Input side of the time-mix layer (rwkv6_model.py:134-146): what the layer does to its input x
// before the projections that produce the operator's r, k, v, w and the gate.
//
//   xx    = shift(x) - x                     previous token (zero before the first) minus the token, :40-43
//   x_mix = x + xx * mix_x                                                                           :136
//   h_s   = tanh(x_mix A_s^T)                five low-rank mixers (DecomposerDense, :11-25), s = r,k,v,w,g;
//   coef_s = h_s W_s^T + bias_s              rank R = decomposer_size                                :139
//   x_s   = x + xx * coef_s                                                                          :141-145
//
// The two GEMMs against A (hidden -> 5R) stay with the caller's GEMM library.  The rank-R expansion
// h_s W_s^T is done here, on the matrix cores, inside the kernel that writes the five x_s: one
// 16x16x32 MFMA per 16 tokens x 16 channels and mixer at R = 32, so the five (B,T,C) coefficient
// tensors never exist in memory.  Forward traffic: x in, five tensors out.
//
// Backward, for incoming gradients g_s of the five outputs (coef_s is formed again the same way):
//   gcoef_s = g_s * xx                       written out: the caller's GEMMs reduce it over channels
//                                            (gradient of h_s) and over tokens (gradients of W_s, bias_s)
//   gxx     = sum_s g_s * coef_s             gradient reaching xx through the five outputs
//   gp      = sum_s g_s - gxx                the part of x's gradient that needs no neighbouring token
// and, once the caller has taken gh_s through tanh and A to the gradient gxm of x_mix:
//   z  = gxx + gxm * mix_x                   total gradient of xx
//   gx = gp + gxm * (1 - mix_x) + z[t+1]     (z[t+1] = 0 for the last token of a sequence)
//   gmix_x = sum over tokens of gxm * xx
//
// Layouts: x, outputs and their gradients (B,T,C) 16-bit; h (B,T,5,R); W (5,C,R), i.e. each mixer's
// second weight as a Linear layer stores it (out = C, in = R); bias (5,C) and mix_x (C) fp32.
// MFMA shape D[m][n] = sum_k a[m][k] b[n][k] with a = W rows (m = channel) and b = h rows (n = token):
// lane (n = lane % 16, g = lane / 16) receives rows m = 4g .. 4g+3 of each of a wave's four tiles.
// WHICH channel a row stands for is free (it only decides which row of W is loaded into the operand),
// and is chosen so that a lane's sixteen values are two runs of eight neighbouring channels:
// tile mt, row 4g+e  <->  channel 8 g + 4 mt + e  of the wave's 32 (tiles mt = 0, 1).
// Every tensor is then touched with 16-byte accesses, 64 contiguous bytes per token and instruction.
#include "wkv6_common.h"
#include "wkv6_kernels.h"
#include "wkv6_mfma.h"

namespace wkv6 {

constexpr int kMixers = 5;
constexpr int kMixTiles = 2;       // 16-channel MFMA tiles per wave: 32 channels, 64 contiguous bytes per token
constexpr int kMixWaveCh = 16 * kMixTiles, kMixGroupCh = 4 * kMixWaveCh;   // channels per wave, per workgroup
constexpr int kMixTokBlocks = 8;   // 16-token blocks one workgroup walks through (the W fragments stay in registers)

// what one wave keeps for its channels: the W fragments and the biases of the five mixers
template <int R> struct MixWeights {
    bf16x8 w[kMixers][kMixTiles][R / 32];
    f32x4 b[kMixers][kMixTiles];
    __device__ __forceinline__ void load(const bf16_t *__restrict__ w2t, const float *__restrict__ bias, int C, int c0, int l16, int g) {
#pragma unroll
        for (int s = 0; s < kMixers; ++s)
#pragma unroll
            for (int m = 0; m < kMixTiles; ++m) {
                const int ch = c0 + 8 * (l16 >> 2) + 4 * m + (l16 & 3);
                const bf16_t *row = w2t + ((size_t)s * C + ch) * R + 8 * g;
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) w[s][m][kk] = *reinterpret_cast<const bf16x8 *>(row + 32 * kk);
                const float4 bb = *reinterpret_cast<const float4 *>(bias + (size_t)s * C + c0 + 8 * g + 4 * m);
                b[s][m] = (f32x4){bb.x, bb.y, bb.z, bb.w};
            }
    }
};

// eight consecutive bf16 (tiles 0 and 1 of one lane: element [m][e] belongs to MFMA tile m, row 4g+e)
__device__ __forceinline__ void unpack8(const Raw8<bf16_t> &r, float (&o)[kMixTiles][4]) {
    float f[8];
    r.to_float(f);
#pragma unroll
    for (int e = 0; e < 4; ++e) { o[0][e] = f[e]; o[1][e] = f[4 + e]; }
}
__device__ __forceinline__ void store8(bf16_t *p, const float (&v)[kMixTiles][4]) {
    *reinterpret_cast<uint4 *>(p) = make_uint4(pack_bf16x2(v[0][0], v[0][1]), pack_bf16x2(v[0][2], v[0][3]),
                                               pack_bf16x2(v[1][0], v[1][1]), pack_bf16x2(v[1][2], v[1][3]));
}

// What one wave reads for a block of 16 tokens, as loaded: the kernels fetch block i+1 before they
// work on block i, so a wave always has one block's loads in flight behind its stores.
template <int R, bool kGrads> struct MixBlock {
    bf16x8 hb[kMixers][R / 32];
    Raw8<bf16_t> x, xp, g[kMixers];
    size_t e0;
    bool valid;
    __device__ __forceinline__ void load(int64_t n0, int64_t n_tok, int T, int C, int c0, int l16, int g4,
                                         const bf16_t *__restrict__ xs, const bf16_t *__restrict__ h,
                                         const bf16_t *const (&gs)[kMixers]) {
        const int64_t tok = n0 + l16;
        valid = tok < n_tok;
        const int64_t tc = valid ? tok : n_tok - 1;
        e0 = (size_t)tc * C + c0 + 8 * g4;
#pragma unroll
        for (int s = 0; s < kMixers; ++s)
#pragma unroll
            for (int kk = 0; kk < R / 32; ++kk)
                hb[s][kk] = *reinterpret_cast<const bf16x8 *>(h + ((size_t)tc * kMixers + s) * R + 32 * kk + 8 * g4);
        x.load(xs + e0);
        if (tc % T != 0) xp.load(xs + e0 - C); else xp.zero();
        if (kGrads) {
#pragma unroll
            for (int s = 0; s < kMixers; ++s) g[s].load(gs[s] + e0);
        }
    }
    // x and xx = previous token - x at the lane's channels
    __device__ __forceinline__ void x_and_xx(float (&xv)[kMixTiles][4], float (&xx)[kMixTiles][4]) const {
        unpack8(x, xv);
        unpack8(xp, xx);
#pragma unroll
        for (int m = 0; m < kMixTiles; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) xx[m][e] -= xv[m][e];
    }
};

template <int R>
__global__ __launch_bounds__(256) void shift_mix5_fwd_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const bf16_t *__restrict__ h, const bf16_t *__restrict__ w2t, const float *__restrict__ bias,
        bf16_t *__restrict__ o0, bf16_t *__restrict__ o1, bf16_t *__restrict__ o2, bf16_t *__restrict__ o3, bf16_t *__restrict__ o4)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, g = lane >> 4;
    const int ncg = (C + kMixGroupCh - 1) / kMixGroupCh;   // workgroups side by side over the channels: neighbours share token rows
    const int c0 = ((int)(blockIdx.x % ncg) * 4 + wave) * kMixWaveCh;
    const int64_t first = (int64_t)(blockIdx.x / ncg) * (16 * kMixTokBlocks);
    if (c0 >= C || first >= n_tok) return;
    MixWeights<R> wt;
    wt.load(w2t, bias, C, c0, l16, g);
    bf16_t *const outs[kMixers] = {o0, o1, o2, o3, o4};
    const bf16_t *const none[kMixers] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    MixBlock<R, false> cur, nxt;
    cur.load(first, n_tok, T, C, c0, l16, g, x, h, none);
    for (int tb = 0; tb < kMixTokBlocks; ++tb) {
        const int64_t n1 = first + 16 * (tb + 1);
        const bool more = tb + 1 < kMixTokBlocks && n1 < n_tok;
        if (more) nxt.load(n1, n_tok, T, C, c0, l16, g, x, h, none);
        float xv[kMixTiles][4], xx[kMixTiles][4];
        cur.x_and_xx(xv, xx);
#pragma unroll
        for (int s = 0; s < kMixers; ++s) {
            float o[kMixTiles][4];
#pragma unroll
            for (int m = 0; m < kMixTiles; ++m) {
                f32x4 acc = wt.b[s][m];
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) acc = mfma32(wt.w[s][m][kk], cur.hb[s][kk], acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[m][e] = fmaf(xx[m][e], acc[e], xv[m][e]);
            }
            if (cur.valid) store8(outs[s] + cur.e0, o);
        }
        if (!more) break;
        cur = nxt;
    }
}

template <int R>
__global__ __launch_bounds__(256) void shift_mix5_bwd_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const bf16_t *__restrict__ h, const bf16_t *__restrict__ w2t, const float *__restrict__ bias,
        const bf16_t *__restrict__ g0, const bf16_t *__restrict__ g1, const bf16_t *__restrict__ g2, const bf16_t *__restrict__ g3,
        const bf16_t *__restrict__ g4, bf16_t *__restrict__ gcoef, int64_t plane, bf16_t *__restrict__ gp, bf16_t *__restrict__ gxx)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, g = lane >> 4;
    const int ncg = (C + kMixGroupCh - 1) / kMixGroupCh;   // workgroups side by side over the channels: neighbours share token rows
    const int c0 = ((int)(blockIdx.x % ncg) * 4 + wave) * kMixWaveCh;
    const int64_t first = (int64_t)(blockIdx.x / ncg) * (16 * kMixTokBlocks);
    if (c0 >= C || first >= n_tok) return;
    MixWeights<R> wt;
    wt.load(w2t, bias, C, c0, l16, g);
    const bf16_t *const gs[kMixers] = {g0, g1, g2, g3, g4};
    MixBlock<R, true> cur, nxt;
    cur.load(first, n_tok, T, C, c0, l16, g, x, h, gs);
    for (int tb = 0; tb < kMixTokBlocks; ++tb) {
        const int64_t n1 = first + 16 * (tb + 1);
        const bool more = tb + 1 < kMixTokBlocks && n1 < n_tok;
        if (more) nxt.load(n1, n_tok, T, C, c0, l16, g, x, h, gs);
        float xv[kMixTiles][4], xx[kMixTiles][4];
        cur.x_and_xx(xv, xx);
        float sum[kMixTiles][4], sxx[kMixTiles][4];
#pragma unroll
        for (int m = 0; m < kMixTiles; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) { sum[m][e] = 0.f; sxx[m][e] = 0.f; }
#pragma unroll
        for (int s = 0; s < kMixers; ++s) {
            float gg[kMixTiles][4], gc[kMixTiles][4];
            unpack8(cur.g[s], gg);
#pragma unroll
            for (int m = 0; m < kMixTiles; ++m) {
                f32x4 acc = wt.b[s][m];
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) acc = mfma32(wt.w[s][m][kk], cur.hb[s][kk], acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sum[m][e] += gg[m][e];
                    sxx[m][e] = fmaf(gg[m][e], acc[e], sxx[m][e]);
                    gc[m][e] = gg[m][e] * xx[m][e];
                }
            }
            if (cur.valid) store8(gcoef + s * plane + cur.e0, gc);
        }
        if (cur.valid) {
#pragma unroll
            for (int m = 0; m < kMixTiles; ++m)
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[m][e] -= sxx[m][e];
            store8(gxx + cur.e0, sxx);
            store8(gp + cur.e0, sum);
        }
        if (!more) break;
        cur = nxt;
    }
}

constexpr int kMixXRun = 4;   // consecutive tokens per thread of the kernel below

// x_mix = x + xx * mix_x: one thread per 8 channels of four consecutive tokens (each row of x is
// fetched once, plus one row in four for the token before the run)
__global__ __launch_bounds__(256) void shift_mix_x_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const float *__restrict__ mix_x, bf16_t *__restrict__ x_mix)
{
    const int per_row = C / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t run = i / per_row, tok0 = run * kMixXRun;
    if (tok0 >= n_tok) return;
    const int c = (int)(i - run * per_row) * 8;
    float mx[8], xp[8];
    Raw8<float> m8;
    m8.load(mix_x + c);
    m8.to_float(mx);
    Raw8<bf16_t> rows[kMixXRun], p;
    if (tok0 % T != 0) p.load(x + (size_t)(tok0 - 1) * C + c); else p.zero();
#pragma unroll
    for (int j = 0; j < kMixXRun; ++j)
        if (tok0 + j < n_tok) rows[j].load(x + (size_t)(tok0 + j) * C + c); else rows[j].zero();
    p.to_float(xp);
#pragma unroll
    for (int j = 0; j < kMixXRun; ++j) {
        float xa[8], o[8];
        rows[j].to_float(xa);
        const bool first = (tok0 + j) % T == 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) { o[q] = fmaf((first ? 0.f : xp[q]) - xa[q], mx[q], xa[q]); xp[q] = xa[q]; }
        if (tok0 + j < n_tok)
            *reinterpret_cast<uint4 *>(x_mix + (size_t)(tok0 + j) * C + c) =
                make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    }
}

constexpr int kMixRows = 8;        // token rows a workgroup of the kernel below works on at once
constexpr int kMixRun = 64;        // tokens per workgroup

// gx = gp + gxm (1 - mix_x) + z[t+1],  z = gxx + gxm mix_x;  gmix_x += gxm * xx.
// gp and gxx may be null (both zero): the backward of x_mix = x + xx * mix_x on its own.
// Thread (row, column group): 8 channels of every 8th token of the workgroup's 64 tokens; the
// per-channel sums go through LDS to one atomic per channel and workgroup.
__global__ __launch_bounds__(256) void shift_mix_x_bwd_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const float *__restrict__ mix_x, const bf16_t *__restrict__ gp, const bf16_t *__restrict__ gxx,
        const bf16_t *__restrict__ gxm, bf16_t *__restrict__ gx, float *__restrict__ gmix_x)
{
    __shared__ float part[kMixRows][256 + 8];
    const int col = threadIdx.x & 31, row = threadIdx.x >> 5;
    const int ncg = (C + 255) / 256, cg = (int)(blockIdx.x % ncg);
    const int c = (cg * 32 + col) * 8;
    const bool live = c < C;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
        float mx[8];
        Raw8<float> m8;
        m8.load(mix_x + c);
        m8.to_float(mx);
        const int64_t first = (int64_t)(blockIdx.x / ncg) * kMixRun;
        for (int it = 0; it < kMixRun / kMixRows; ++it) {
            const int64_t tok = first + it * kMixRows + row;
            if (tok >= n_tok) break;
            const size_t e = (size_t)tok * C + c;
            const int t = (int)(tok % T);
            Raw8<bf16_t> rx, rp, rg, rm, rzn, rmn;
            rx.load(x + e); rm.load(gxm + e);
            if (gp) rg.load(gp + e); else rg.zero();
            if (t != 0) rp.load(x + e - C); else rp.zero();
            if (t != T - 1) { rmn.load(gxm + e + C); if (gxx) rzn.load(gxx + e + C); else rzn.zero(); } else { rzn.zero(); rmn.zero(); }
            float xa[8], xp[8], p[8], m[8], zn[8], mn[8], o[8];
            rx.to_float(xa); rp.to_float(xp); rg.to_float(p); rm.to_float(m); rzn.to_float(zn); rmn.to_float(mn);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                o[j] = p[j] + m[j] * (1.f - mx[j]) + fmaf(mn[j], mx[j], zn[j]);
                acc[j] = fmaf(m[j], xp[j] - xa[j], acc[j]);
            }
            *reinterpret_cast<uint4 *>(gx + e) = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) part[row][col * 8 + j] = acc[j];
    __syncthreads();
    const int cc = cg * 256 + threadIdx.x;
    if (cc < C) {
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < kMixRows; ++r) s += part[r][threadIdx.x];
        atomicAdd(gmix_x + cc, s);
    }
}

__global__ void zero1_kernel(int n, float *a) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a[i] = 0.f;
}

bool shift_mix_supported(int64_t C, int64_t R) { return C > 0 && C % 64 == 0 && (R == 32 || R == 64); }

static dim3 mix5_grid(int64_t n_tok, int64_t C) {
    return dim3((unsigned)(((C + kMixGroupCh - 1) / kMixGroupCh) * ((n_tok + 16 * kMixTokBlocks - 1) / (16 * kMixTokBlocks))));
}

hipError_t shift_mix_x(hipStream_t st, int64_t B, int64_t T, int64_t C, const void *x, const float *mix_x, void *x_mix) {
    const int64_t n = B * T, threads = (n + kMixXRun - 1) / kMixXRun * (C / 8);
    hipLaunchKernelGGL(shift_mix_x_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, n, (int)T, (int)C,
                       (const bf16_t *)x, mix_x, (bf16_t *)x_mix);
    return hipGetLastError();
}

hipError_t shift_mix_five(hipStream_t st, int64_t B, int64_t T, int64_t C, int64_t R, const void *x, const void *h,
                          const void *w2t, const float *bias, void *const out[5]) {
    const int64_t n = B * T;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, mix5_grid(n, C), dim3(256), 0, st, n, (int)T, (int)C, (const bf16_t *)x, (const bf16_t *)h,
                           (const bf16_t *)w2t, bias, (bf16_t *)out[0], (bf16_t *)out[1], (bf16_t *)out[2], (bf16_t *)out[3], (bf16_t *)out[4]);
    };
    if (R == 32) launch(shift_mix5_fwd_kernel<32>); else launch(shift_mix5_fwd_kernel<64>);
    return hipGetLastError();
}

hipError_t shift_mix_five_backward(hipStream_t st, int64_t B, int64_t T, int64_t C, int64_t R, const void *x, const void *h,
                                   const void *w2t, const float *bias, const void *const gout[5], void *gcoef, int64_t gcoef_stride,
                                   void *gp, void *gxx) {
    const int64_t n = B * T;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, mix5_grid(n, C), dim3(256), 0, st, n, (int)T, (int)C, (const bf16_t *)x, (const bf16_t *)h,
                           (const bf16_t *)w2t, bias, (const bf16_t *)gout[0], (const bf16_t *)gout[1], (const bf16_t *)gout[2],
                           (const bf16_t *)gout[3], (const bf16_t *)gout[4], (bf16_t *)gcoef, gcoef_stride, (bf16_t *)gp, (bf16_t *)gxx);
    };
    if (R == 32) launch(shift_mix5_bwd_kernel<32>); else launch(shift_mix5_bwd_kernel<64>);
    return hipGetLastError();
}

hipError_t shift_mix_x_backward(hipStream_t st, int64_t B, int64_t T, int64_t C, const void *x, const float *mix_x,
                                const void *gp, const void *gxx, const void *gxm, void *gx, float *gmix_x) {
    const int64_t n = B * T;
    // (a fill kernel rather than a memset node: the call may be captured in a HIP graph)
    hipLaunchKernelGGL(zero1_kernel, dim3((unsigned)((C + 255) / 256)), dim3(256), 0, st, (int)C, gmix_x);
    hipLaunchKernelGGL(shift_mix_x_bwd_kernel, dim3((unsigned)(((C + 255) / 256) * ((n + kMixRun - 1) / kMixRun))), dim3(256), 0, st,
                       n, (int)T, (int)C, (const bf16_t *)x, mix_x, (const bf16_t *)gp, (const bf16_t *)gxx, (const bf16_t *)gxm,
                       (bf16_t *)gx, gmix_x);
    return hipGetLastError();
}

}  // namespace wkv6
