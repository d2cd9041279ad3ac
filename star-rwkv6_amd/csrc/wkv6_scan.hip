// WKV6 as a per-timestep recurrence ("scan") for gfx950.
//
// One workgroup per (batch, head).  The 64x64 fp32 state lives in VGPRs, split over the
// workgroup's waves (16 state values per lane); tiles of TC timesteps of the inputs are staged
// through LDS as fp32 with 16-byte coalesced global loads that are issued one tile ahead and
// parked in registers while the current tile is consumed.  All arithmetic is fp32, one rounding
// on store, like the reference kernels (rwkv_kernel/jax_kernel/rwkv_kernels.cu:107-160 forward,
// :205-407 backward) -- but the mapping is different: the reference runs one 64-thread block
// with the whole state column per thread; here 4, 8 or 16 waves share a head, operands that are
// uniform over a wave come from LDS broadcast reads, and cross-wave sums go through LDS once
// per tile instead of two barriers per timestep.
//
// This path is exact fp32 and has no restriction on T; it serves fp32 tensors, single-token
// decode and any shape the chunked MFMA path does not take.
#include "wkv6_common.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

namespace wkv6 {

// Sixteen waves per pair, four key rows each: what limits the forward is the LDS read path (every
// wave reads the r, k, d values of its rows as broadcast 16-byte reads, which cost a full 64-lane
// return each), and four waves per SIMD overlap those reads with each other's arithmetic
// (B8 T1024 H32 fp32: 329 us with 4 waves, 295 with 8, 233 with 16).
constexpr int kScanFwdWaves = 16;
template <typename Tin, typename Tout, typename Ts>
__global__ __launch_bounds__(64 * kScanFwdWaves) void scan_fwd_kernel(int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u,
        const Ts *__restrict__ s0, const int64_t *__restrict__ map,
        Tout *__restrict__ y, Ts *__restrict__ sT)
{
    extern __shared__ __align__(16) unsigned char scan_smem[];
    scan_fwd_body<Tin, Tout, Ts, kScanFwdWaves>(*reinterpret_cast<ScanFwdLdsT<kScanFwdWaves> *>(scan_smem),
                                                blockIdx.x / H, blockIdx.x % H, T, H, r, k, v, w, u, s0, map, y, sT);
}

// One timestep (T = 1: the decode step of a served model).  Nothing is carried inside the kernel, so
// a pair needs no workgroup: one wave per (batch, head), four pairs per workgroup, no LDS, no
// barrier.  Lane l owns value columns 4 (l & 15) .. +3 of key rows 16 (l >> 4) .. +15: the state
// streams through as sixteen 16-byte loads and stores per lane, all issued at once, and y is
// folded over the four row groups with two wavefront shuffles per value.
// kFuse: y is replaced by (layer_norm(y over the head's 64 channels, eps) * gn_scale + gn_offset) * gate,
// the model's next two steps (the 64 values of a head sit in 16 lanes of the wave).
template <typename Tin, typename Tout, typename Ts, bool kFuse>
__global__ __launch_bounds__(256) void step_fwd_kernel(int npairs, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u,
        const Ts *__restrict__ s0, const int64_t *__restrict__ map,
        Tout *__restrict__ y, Ts *__restrict__ sT,
        const Tin *__restrict__ gate, const float *__restrict__ gn_scale, const float *__restrict__ gn_offset, float gn_eps)
{
    const int lane = threadIdx.x & 63;
    const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pair >= npairs) return;
    const int b = pair / H, h = pair - b * H;
    const int i4 = (lane & 15) * 4, j0 = (lane >> 4) * 16;
    const int64_t tok = (int64_t)pair * kN;   // T = 1: (b, 0, h*64) is element pair*64 of a (B,1,C) tensor
    float S[16][4];
    if (s0) {
        const int64_t row = map ? map[b] : (int64_t)b;
        const Ts *p = s0 + ((row * H + h) * kN + j0) * kN + i4;
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) load4(p + jj * kN, S[jj]);
    } else {
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) S[jj][0] = S[jj][1] = S[jj][2] = S[jj][3] = 0.f;
    }
    Raw8<Tin> rr[2], rk[2], rw[2], ru[2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        rr[x].load(r + tok + j0 + 8 * x); rk[x].load(k + tok + j0 + 8 * x);
        rw[x].load(w + tok + j0 + 8 * x); ru[x].load(u + h * kN + j0 + 8 * x);
    }
    float vv[4];
    load4(v + tok + i4, vv);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        float fr[8], fk[8], fw[8], fu[8];
        rr[x].to_float(fr); rk[x].to_float(fk); rw[x].to_float(fw); ru[x].to_float(fu);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float d = decay_from_raw(fw[e]), uk = fu[e] * fk[e];
            float (&Sj)[4] = S[8 * x + e];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                acc[c] = fmaf(fr[e], fmaf(uk, vv[c], Sj[c]), acc[c]);
                Sj[c] = fmaf(Sj[c], d, fk[e] * vv[c]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        acc[c] += __shfl_xor(acc[c], 16);
        acc[c] += __shfl_xor(acc[c], 32);
    }
    if (kFuse) {
        // every lane holds the y of its 4 columns; fold mean and variance over the 16 column groups
        float sum = (acc[0] + acc[1]) + (acc[2] + acc[3]);
#pragma unroll
        for (int m = 8; m >= 1; m >>= 1) sum += __shfl_xor(sum, m);
        const float mu = sum * (1.f / kN);
        float d[4], sq = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) { d[c] = acc[c] - mu; sq = fmaf(d[c], d[c], sq); }
#pragma unroll
        for (int m = 8; m >= 1; m >>= 1) sq += __shfl_xor(sq, m);
        const float rstd = __builtin_amdgcn_rsqf(sq * (1.f / kN) + gn_eps);
        float gt[4], sc[4], of[4];
        load4(gate + tok + i4, gt);
        load4(gn_scale + h * kN + i4, sc);
        load4(gn_offset + h * kN + i4, of);
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] = fmaf(d[c] * rstd, sc[c], of[c]) * gt[c];
    }
    if (lane < 16) store4(y + tok + i4, acc[0], acc[1], acc[2], acc[3]);
    if (sT) {
        Ts *p = sT + ((int64_t)pair * kN + j0) * kN + i4;
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) store4(p + jj * kN, S[jj][0], S[jj][1], S[jj][2], S[jj][3]);
    }
}

constexpr int kScanBwdAWaves = 16;   // four value columns per wave, for the same reason as in the forward
template <typename Tin, typename Tout>
__global__ __launch_bounds__(64 * kScanBwdAWaves) void scan_bwd_a_kernel(int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u, const Tout *__restrict__ gy,
        Tout *__restrict__ gr, Tout *__restrict__ gu, float *__restrict__ wsP,
        const float *__restrict__ s0, const float *__restrict__ gsT, float *__restrict__ fT)
{
    extern __shared__ __align__(16) unsigned char scan_smem[];
    auto &lds = *reinterpret_cast<ScanBwdALdsT<kScanBwdAWaves> *>(scan_smem);
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t C = (int64_t)H * kN;
    const int64_t pair = blockIdx.x;
    scan_bwd_a_body<Tin, Tout, kScanBwdAWaves>(lds, b, h, T, H, r, k, v, w, u, gy, gr, gu, wsP + (int64_t)b * T * C + h * kN, C,
                               s0 ? s0 + pair * kN * kN : nullptr, gsT ? gsT + pair * kN * kN : nullptr,
                               fT ? fT + pair * kN : nullptr);
}

constexpr int kScanBwdBRoleWaves = 4;   // waves per role (8 in all), sixteen columns / rows each (8 per role: registers spill, 1.5 % faster)
template <typename Tin, typename Tout>
__global__ __launch_bounds__(128 * kScanBwdBRoleWaves) void scan_bwd_b_kernel(int T, int H,
        const Tin *__restrict__ r, const Tin *__restrict__ k, const Tin *__restrict__ v,
        const Tin *__restrict__ w, const Tin *__restrict__ u, const Tout *__restrict__ gy,
        const float *__restrict__ wsP,
        Tout *__restrict__ gk, Tout *__restrict__ gv, Tout *__restrict__ gw,
        const float *__restrict__ gsT, const float *__restrict__ fT, float *__restrict__ gs0, int first_decay_unused)
{
    extern __shared__ __align__(16) unsigned char scan_smem[];
    auto &lds = *reinterpret_cast<ScanBwdBLdsT<kScanBwdBRoleWaves> *>(scan_smem);
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t C = (int64_t)H * kN;
    const int64_t pair = blockIdx.x;
    scan_bwd_b_body<Tin, Tout, kScanBwdBRoleWaves>(lds, b, h, T, H, r, k, v, w, u, gy, wsP + (int64_t)b * T * C + h * kN, C, gk, gv, gw,
                               gsT ? gsT + pair * kN * kN : nullptr, fT ? fT + pair * kN : nullptr,
                               gs0 ? gs0 + pair * kN * kN : nullptr, first_decay_unused != 0);
}

// ------------------------------------------------------------------------------------------
// host launchers
// ------------------------------------------------------------------------------------------
template <typename Tin, typename Tout, typename Ts>
static hipError_t launch_fwd(hipStream_t st, int64_t B, int64_t T, int64_t H, const void *r, const void *k,
                             const void *v, const void *w, const void *u, const void *s0, const int64_t *map,
                             void *y, void *sT)
{
    if (T == 1) {
        hipLaunchKernelGGL((step_fwd_kernel<Tin, Tout, Ts, false>), dim3((unsigned)((B * H + 3) / 4)), dim3(256), 0, st, (int)(B * H), (int)H,
                           (const Tin *)r, (const Tin *)k, (const Tin *)v, (const Tin *)w, (const Tin *)u,
                           (const Ts *)s0, map, (Tout *)y, (Ts *)sT, (const Tin *)nullptr, (const float *)nullptr, (const float *)nullptr, 0.f);
        return hipGetLastError();
    }
    constexpr int lds = (int)sizeof(ScanFwdLdsT<kScanFwdWaves>);
    const hipError_t e = allow_dynamic_lds<scan_fwd_kernel<Tin, Tout, Ts>>(lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, Ts>), dim3((unsigned)(B * H)), dim3(64 * kScanFwdWaves), lds, st, (int)T, (int)H,
                       (const Tin *)r, (const Tin *)k, (const Tin *)v, (const Tin *)w, (const Tin *)u,
                       (const Ts *)s0, map, (Tout *)y, (Ts *)sT);
    return hipGetLastError();
}

hipError_t scan_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H,
                        const void *r, const void *k, const void *v, const void *w, const void *u,
                        const void *s0, const int64_t *map, void *y, void *sT)
{
    const bool sf32 = (state_dtype == kF32);
    switch (dtype) {
    case kF32: return launch_fwd<float, float, float>(st, B, T, H, r, k, v, w, u, s0, map, y, sT);
    case kF16: return launch_fwd<f16_t, float, float>(st, B, T, H, r, k, v, w, u, s0, map, y, sT);
    default:
        return sf32 ? launch_fwd<bf16_t, bf16_t, float>(st, B, T, H, r, k, v, w, u, s0, map, y, sT)
                    : launch_fwd<bf16_t, bf16_t, bf16_t>(st, B, T, H, r, k, v, w, u, s0, map, y, sT);
    }
}

// single timestep with the fused output stage (bf16 tensors)
hipError_t step_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t H,
                              const void *r, const void *k, const void *v, const void *w, const void *u,
                              const void *s0, const int64_t *map, const void *gate, const float *gn_scale,
                              const float *gn_offset, float gn_eps, void *out, void *sT)
{
    const dim3 grid((unsigned)((B * H + 3) / 4)), block(256);
    if (state_dtype == kF32)
        hipLaunchKernelGGL((step_fwd_kernel<bf16_t, bf16_t, float, true>), grid, block, 0, st, (int)(B * H), (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const float *)s0, map, (bf16_t *)out, (float *)sT, (const bf16_t *)gate, gn_scale, gn_offset, gn_eps);
    else
        hipLaunchKernelGGL((step_fwd_kernel<bf16_t, bf16_t, bf16_t, true>), grid, block, 0, st, (int)(B * H), (int)H,
                           (const bf16_t *)r, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)w, (const bf16_t *)u,
                           (const bf16_t *)s0, map, (bf16_t *)out, (bf16_t *)sT, (const bf16_t *)gate, gn_scale, gn_offset, gn_eps);
    return hipGetLastError();
}

template <typename Tin, typename Tout>
static hipError_t launch_bwd(hipStream_t st, int64_t B, int64_t T, int64_t H, const void *r, const void *k,
                             const void *v, const void *w, const void *u, const void *gy, void *gr, void *gk,
                             void *gv, void *gw, void *gu, float *wsP,
                             const float *s0 = nullptr, const float *gsT = nullptr, float *gs0 = nullptr)
{
    // with state gradients: F_T (one value per channel and batch row) sits behind P in the workspace
    float *fT = (s0 || gsT || gs0) ? wsP + B * T * H * kN : nullptr;
    constexpr int lds_a = (int)sizeof(ScanBwdALdsT<kScanBwdAWaves>);
    hipError_t e = allow_dynamic_lds<scan_bwd_a_kernel<Tin, Tout>>(lds_a);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((scan_bwd_a_kernel<Tin, Tout>), dim3((unsigned)(B * H)), dim3(64 * kScanBwdAWaves), lds_a, st, (int)T, (int)H,
                       (const Tin *)r, (const Tin *)k, (const Tin *)v, (const Tin *)w, (const Tin *)u,
                       (const Tout *)gy, (Tout *)gr, (Tout *)gu, wsP, s0, gsT, fT);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    constexpr int lds_b = (int)sizeof(ScanBwdBLdsT<kScanBwdBRoleWaves>);
    e = allow_dynamic_lds<scan_bwd_b_kernel<Tin, Tout>>(lds_b);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((scan_bwd_b_kernel<Tin, Tout>), dim3((unsigned)(B * H)), dim3(128 * kScanBwdBRoleWaves), lds_b, st, (int)T, (int)H,
                       (const Tin *)r, (const Tin *)k, (const Tin *)v, (const Tin *)w, (const Tin *)u,
                       (const Tout *)gy, (const float *)wsP, (Tout *)gk, (Tout *)gv, (Tout *)gw,
                       gsT, (const float *)fT, gs0, s0 ? 0 : 1);
    return hipGetLastError();
}

size_t scan_backward_workspace_bytes(int64_t B, int64_t T, int64_t C) { return (size_t)(B * T * C) * sizeof(float); }
size_t scan_backward_state_workspace_bytes(int64_t B, int64_t T, int64_t C) {
    return (size_t)(B * T * C + B * C) * sizeof(float);
}

hipError_t scan_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace)
{
    float *wsP = (float *)workspace;
    switch (dtype) {
    case kF32: return launch_bwd<float, float>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP);
    case kF16: return launch_bwd<f16_t, float>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP);
    default:   return launch_bwd<bf16_t, bf16_t>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP);
    }
}

hipError_t scan_backward_state(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const float *s0, const void *gy, const float *gsT,
                               void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0, void *workspace)
{
    float *wsP = (float *)workspace;
    switch (dtype) {
    case kF32: return launch_bwd<float, float>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP, s0, gsT, gs0);
    case kF16: return launch_bwd<f16_t, float>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP, s0, gsT, gs0);
    default:   return launch_bwd<bf16_t, bf16_t>(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, wsP, s0, gsT, gs0);
    }
}

}  // namespace wkv6
