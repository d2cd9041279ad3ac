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
// tile mt, row 4g+e  <->  channel 32 (mt / 2) + 8 g + 4 (mt % 2) + e  of the wave's 64.
// Every tensor is then touched with 16-byte accesses, 64 contiguous bytes per token and instruction.
#include "wkv6_common.h"
#include "wkv6_kernels.h"
#include "wkv6_mfma.h"

namespace wkv6 {

constexpr int kMixers = 5;
constexpr int kMixTokBlocks = 8;   // 16-token blocks one workgroup walks through (the W fragments stay in registers)

// what one wave keeps for its 64 channels: the W fragments and the biases of the five mixers
template <int R> struct MixWeights {
    bf16x8 w[kMixers][4][R / 32];
    f32x4 b[kMixers][4];
    __device__ __forceinline__ void load(const bf16_t *__restrict__ w2t, const float *__restrict__ bias, int C, int c0, int l16, int g) {
#pragma unroll
        for (int s = 0; s < kMixers; ++s)
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const int ch = c0 + 32 * (m >> 1) + 8 * (l16 >> 2) + 4 * (m & 1) + (l16 & 3);
                const bf16_t *row = w2t + ((size_t)s * C + ch) * R + 8 * g;
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) w[s][m][kk] = *reinterpret_cast<const bf16x8 *>(row + 32 * kk);
                const float4 bb = *reinterpret_cast<const float4 *>(bias + (size_t)s * C + c0 + 32 * (m >> 1) + 8 * g + 4 * (m & 1));
                b[s][m] = (f32x4){bb.x, bb.y, bb.z, bb.w};
            }
    }
};

// A lane's sixteen channels of one token: element [m][e] belongs to MFMA tile m, row 4g+e; in memory
// two runs of eight, at offsets 0 and 32 from the lane's first channel.
__device__ __forceinline__ void load16(const bf16_t *__restrict__ p, float (&o)[4][4]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        Raw8<bf16_t> r;
        float f[8];
        r.load(p + 32 * j);
        r.to_float(f);
#pragma unroll
        for (int e = 0; e < 4; ++e) { o[2 * j][e] = f[e]; o[2 * j + 1][e] = f[4 + e]; }
    }
}
// eight values (tiles 2j and 2j+1 of one lane) as one 16-byte store
__device__ __forceinline__ void store8(bf16_t *p, const float (&lo)[4], const float (&hi)[4]) {
    *reinterpret_cast<uint4 *>(p) = make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]),
                                               pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]));
}

// x and xx of one lane's token at its 16 channels
struct MixX {
    float x[4][4], xx[4][4];
    __device__ __forceinline__ void load(const bf16_t *__restrict__ xrow, bool has_prev, int C) {
        load16(xrow, x);
        if (has_prev) {
            load16(xrow - C, xx);
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int e = 0; e < 4; ++e) xx[m][e] -= x[m][e];
        } else {
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int e = 0; e < 4; ++e) xx[m][e] = -x[m][e];
        }
    }
};

template <int R>
__global__ __launch_bounds__(256) void shift_mix5_fwd_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const bf16_t *__restrict__ h, const bf16_t *__restrict__ w2t, const float *__restrict__ bias,
        bf16_t *__restrict__ o0, bf16_t *__restrict__ o1, bf16_t *__restrict__ o2, bf16_t *__restrict__ o3, bf16_t *__restrict__ o4)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, g = lane >> 4;
    const int ncg = (C + 255) / 256;   // workgroups side by side over the channels: neighbours share token rows
    const int c0 = ((int)(blockIdx.x % ncg) * 4 + wave) * 64;
    if (c0 >= C) return;
    MixWeights<R> wt;
    wt.load(w2t, bias, C, c0, l16, g);
    bf16_t *const outs[kMixers] = {o0, o1, o2, o3, o4};
    const int64_t first = (int64_t)(blockIdx.x / ncg) * (16 * kMixTokBlocks);
    for (int tb = 0; tb < kMixTokBlocks; ++tb) {
        const int64_t n0 = first + 16 * tb;
        if (n0 >= n_tok) break;
        const int64_t tok = n0 + l16;
        const bool valid = tok < n_tok;
        const int64_t tc = valid ? tok : n_tok - 1;
        const size_t e0 = (size_t)tc * C + c0 + 8 * g;
        bf16x8 hb[kMixers][R / 32];
#pragma unroll
        for (int s = 0; s < kMixers; ++s)
#pragma unroll
            for (int kk = 0; kk < R / 32; ++kk)
                hb[s][kk] = *reinterpret_cast<const bf16x8 *>(h + ((size_t)tc * kMixers + s) * R + 32 * kk + 8 * g);
        MixX xs;
        xs.load(x + e0, tc % T != 0, C);
#pragma unroll
        for (int s = 0; s < kMixers; ++s) {
            float o[4][4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                f32x4 acc = wt.b[s][m];
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) acc = mfma32(wt.w[s][m][kk], hb[s][kk], acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[m][e] = fmaf(xs.xx[m][e], acc[e], xs.x[m][e]);
            }
            if (valid) {
                store8(outs[s] + e0, o[0], o[1]);
                store8(outs[s] + e0 + 32, o[2], o[3]);
            }
        }
    }
}

template <int R>
__global__ __launch_bounds__(256) void shift_mix5_bwd_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const bf16_t *__restrict__ h, const bf16_t *__restrict__ w2t, const float *__restrict__ bias,
        const bf16_t *__restrict__ g0, const bf16_t *__restrict__ g1, const bf16_t *__restrict__ g2, const bf16_t *__restrict__ g3,
        const bf16_t *__restrict__ g4, bf16_t *__restrict__ gcoef, bf16_t *__restrict__ gp, bf16_t *__restrict__ gxx)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l16 = lane & 15, g = lane >> 4;
    const int ncg = (C + 255) / 256;   // workgroups side by side over the channels: neighbours share token rows
    const int c0 = ((int)(blockIdx.x % ncg) * 4 + wave) * 64;
    if (c0 >= C) return;
    MixWeights<R> wt;
    wt.load(w2t, bias, C, c0, l16, g);
    const bf16_t *const gs[kMixers] = {g0, g1, g2, g3, g4};
    const size_t plane = (size_t)n_tok * C;   // one mixer's (B,T,C) slice of gcoef
    const int64_t first = (int64_t)(blockIdx.x / ncg) * (16 * kMixTokBlocks);
    for (int tb = 0; tb < kMixTokBlocks; ++tb) {
        const int64_t n0 = first + 16 * tb;
        if (n0 >= n_tok) break;
        const int64_t tok = n0 + l16;
        const bool valid = tok < n_tok;
        const int64_t tc = valid ? tok : n_tok - 1;
        const size_t e0 = (size_t)tc * C + c0 + 8 * g;
        bf16x8 hb[kMixers][R / 32];
#pragma unroll
        for (int s = 0; s < kMixers; ++s)
#pragma unroll
            for (int kk = 0; kk < R / 32; ++kk)
                hb[s][kk] = *reinterpret_cast<const bf16x8 *>(h + ((size_t)tc * kMixers + s) * R + 32 * kk + 8 * g);
        MixX xs;
        xs.load(x + e0, tc % T != 0, C);
        float sum[4][4], sxx[4][4];
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) { sum[m][e] = 0.f; sxx[m][e] = 0.f; }
#pragma unroll
        for (int s = 0; s < kMixers; ++s) {
            float gg[4][4], gc[4][4];
            load16(gs[s] + e0, gg);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                f32x4 acc = wt.b[s][m];
#pragma unroll
                for (int kk = 0; kk < R / 32; ++kk) acc = mfma32(wt.w[s][m][kk], hb[s][kk], acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sum[m][e] += gg[m][e];
                    sxx[m][e] = fmaf(gg[m][e], acc[e], sxx[m][e]);
                    gc[m][e] = gg[m][e] * xs.xx[m][e];
                }
            }
            if (valid) {
                store8(gcoef + s * plane + e0, gc[0], gc[1]);
                store8(gcoef + s * plane + e0 + 32, gc[2], gc[3]);
            }
        }
        if (valid) {
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int e = 0; e < 4; ++e) sum[m][e] -= sxx[m][e];
            store8(gxx + e0, sxx[0], sxx[1]);
            store8(gxx + e0 + 32, sxx[2], sxx[3]);
            store8(gp + e0, sum[0], sum[1]);
            store8(gp + e0 + 32, sum[2], sum[3]);
        }
    }
}

// x_mix = x + xx * mix_x: one thread per token and 8 channels
__global__ __launch_bounds__(256) void shift_mix_x_kernel(int64_t n_tok, int T, int C,
        const bf16_t *__restrict__ x, const float *__restrict__ mix_x, bf16_t *__restrict__ x_mix)
{
    const int per_row = C / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_tok * per_row) return;
    const int64_t tok = i / per_row;
    const int c = (int)(i - tok * per_row) * 8;
    const size_t e = (size_t)tok * C + c;
    Raw8<bf16_t> a, p;
    a.load(x + e);
    if (tok % T != 0) p.load(x + e - C); else p.zero();
    float xa[8], xp[8], mx[8], o[8];
    a.to_float(xa); p.to_float(xp);
    Raw8<float> m8;
    m8.load(mix_x + c);
    m8.to_float(mx);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = fmaf(xp[j] - xa[j], mx[j], xa[j]);
    *reinterpret_cast<uint4 *>(x_mix + e) = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
}

constexpr int kMixRows = 8;        // token rows a workgroup of the kernel below works on at once
constexpr int kMixRun = 64;        // tokens per workgroup

// gx = gp + gxm (1 - mix_x) + z[t+1],  z = gxx + gxm mix_x;  gmix_x += gxm * xx.
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
            rx.load(x + e); rg.load(gp + e); rm.load(gxm + e);
            if (t != 0) rp.load(x + e - C); else rp.zero();
            if (t != T - 1) { rzn.load(gxx + e + C); rmn.load(gxm + e + C); } else { rzn.zero(); rmn.zero(); }
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
    return dim3((unsigned)(((C + 255) / 256) * ((n_tok + 16 * kMixTokBlocks - 1) / (16 * kMixTokBlocks))));
}

hipError_t shift_mix_x(hipStream_t st, int64_t B, int64_t T, int64_t C, const void *x, const float *mix_x, void *x_mix) {
    const int64_t n = B * T, threads = n * (C / 8);
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
                                   const void *w2t, const float *bias, const void *const gout[5], void *gcoef, void *gp, void *gxx) {
    const int64_t n = B * T;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, mix5_grid(n, C), dim3(256), 0, st, n, (int)T, (int)C, (const bf16_t *)x, (const bf16_t *)h,
                           (const bf16_t *)w2t, bias, (const bf16_t *)gout[0], (const bf16_t *)gout[1], (const bf16_t *)gout[2],
                           (const bf16_t *)gout[3], (const bf16_t *)gout[4], (bf16_t *)gcoef, (bf16_t *)gp, (bf16_t *)gxx);
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
