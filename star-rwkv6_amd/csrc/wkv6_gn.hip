// Backward of the layer's output stage  out = (group_norm_head(y) * scale + offset) * gate  (the forward
// half is fused into the chunked forward kernel, wkv6_chunk_fwd.hip).  group_norm_head is the layer
// norm over one head's 64 channels of one token (rwkv6_model.py:94-99), `* gate` is rwkv6_model.py:158-160.
//
//   z = (y - mean) rstd,  n = z scale + offset,  out = n gate
//   ggate = gout n,  gn = gout gate,  goffset += gn,  gscale += gn z,  gz = gn scale
//   gy = rstd (gz - mean_c(gz) - z mean_c(gz z))          (means over the head's 64 channels)
//
// A (B,T,C) tensor with C = H * 64 is a flat list of B*T*H rows of 64 channels, row i belonging to head
// i % H.  One wave takes rows of ONE head (lane = channel), so the sums for scale and offset stay in
// registers until the wave is done; they are added to the outputs with one atomic per lane and wave.
// Bound by memory: three 16-bit tensors in, two out.
#include "wkv6_common.h"
#include "wkv6_kernels.h"

namespace wkv6 {

__device__ __forceinline__ float wave_sum64(float x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m);
    return x;
}

__global__ __launch_bounds__(256) void gn_gate_bwd_kernel(int64_t rows_per_head, int H,
        const bf16_t *__restrict__ gout, const bf16_t *__restrict__ y, const float *__restrict__ stats,
        const bf16_t *__restrict__ gate, const float *__restrict__ scale, const float *__restrict__ offset,
        bf16_t *__restrict__ gy, bf16_t *__restrict__ ggate, float *__restrict__ gscale, float *__restrict__ goffset)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.x % H;
    const int64_t part = (int64_t)(blockIdx.x / H) * 4 + wave, nparts = (int64_t)(gridDim.x / H) * 4;
    const float sc = scale[h * kN + lane], of = offset[h * kN + lane];
    float acc_s = 0.f, acc_o = 0.f;
    for (int64_t j = part; j < rows_per_head; j += nparts) {
        const int64_t row = j * H + h, e = row * kN + lane;
        const float go = load1(gout + e), yy = load1(y + e), ga = load1(gate + e);
        const float2 st = *reinterpret_cast<const float2 *>(stats + row * 2);
        const float z = (yy - st.x) * st.y;
        const float n = fmaf(z, sc, of);
        const float gn = go * ga;
        store1(ggate + e, go * n);
        acc_o += gn;
        acc_s = fmaf(gn, z, acc_s);
        const float gz = gn * sc;
        const float m1 = wave_sum64(gz) * (1.f / kN), m2 = wave_sum64(gz * z) * (1.f / kN);
        store1(gy + e, st.y * (gz - m1 - z * m2));
    }
    atomicAdd(gscale + h * kN + lane, acc_s);
    atomicAdd(goffset + h * kN + lane, acc_o);
}

__global__ void zero2_kernel(int n, float *a, float *b) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { a[i] = 0.f; b[i] = 0.f; }
}

hipError_t gn_gate_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                            const void *gout, const void *y, const float *stats, const void *gate,
                            const float *scale, const float *offset, void *gy, void *ggate, float *gscale, float *goffset)
{
    const int C = (int)(H * kN);
    // (a fill kernel rather than a memset node: the call may be captured in a HIP graph)
    hipLaunchKernelGGL(zero2_kernel, dim3((unsigned)((C + 255) / 256)), dim3(256), 0, st, C, gscale, goffset);
    const int64_t rows_per_head = B * T;
    // enough waves to fill the chip a few times over, at least a few dozen rows per wave
    int64_t parts = rows_per_head / 4 / 32;
    if (parts < 1) parts = 1;
    const int64_t cap = (4096 + H - 1) / H;
    if (parts > cap) parts = cap;
    hipLaunchKernelGGL(gn_gate_bwd_kernel, dim3((unsigned)(H * parts)), dim3(256), 0, st, rows_per_head, (int)H,
                       (const bf16_t *)gout, (const bf16_t *)y, stats, (const bf16_t *)gate, scale, offset,
                       (bf16_t *)gy, (bf16_t *)ggate, gscale, goffset);
    return hipGetLastError();
}

}  // namespace wkv6
