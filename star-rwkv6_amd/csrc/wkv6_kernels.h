// Host-side launchers of the WKV6 kernels (internal to the library; the public ABI is include/wkv6.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

namespace wkv6 {

// Raises kernel Kern's dynamic-LDS limit to `bytes`, once per device (the setting is idempotent and
// per device; the flags below only save the runtime call on later launches).
template <auto Kern>
inline hipError_t allow_dynamic_lds(int bytes) {
    static std::atomic<bool> done[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool known = dev >= 0 && dev < 64;
    if (known && done[dev].load(std::memory_order_acquire)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && known) done[dev].store(true, std::memory_order_release);
    return e;
}

enum { kBF16 = 0, kF16 = 1, kF32 = 2 };  // same numbering as the public header

// compute units of the current device (an immutable device property, looked up once per device)
int compute_units();

// --- per-timestep recurrence (wkv6_scan.hip) ---
hipError_t scan_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H,
                        const void *r, const void *k, const void *v, const void *w, const void *u,
                        const void *s0, const int64_t *map, void *y, void *sT);
size_t scan_backward_workspace_bytes(int64_t B, int64_t T, int64_t C);
hipError_t scan_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace);

// --- head sizes other than 64, multiples of 4 up to 128 (wkv6_generic.hip): the per-timestep recurrence, one thread per channel; every
// dtype, states (B,H,N,N), state_map, gradients through the state (s0 / gsT / gs0 fp32, may be null)
bool generic_head_size(int64_t N);
hipError_t generic_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                           const void *r, const void *k, const void *v, const void *w, const void *u,
                           const void *s0, const int64_t *map, void *y, void *sT);
size_t generic_backward_workspace_bytes(int64_t B, int64_t T, int64_t C);
hipError_t generic_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const float *s0, const void *gy, const float *gsT,
                            void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0, void *workspace);

// one timestep (T = 1) with the layer's output stage fused in (bf16 tensors), see chunk_forward_fused
hipError_t step_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t H,
                              const void *r, const void *k, const void *v, const void *w, const void *u,
                              const void *s0, const int64_t *map, const void *gate, const float *gn_scale,
                              const float *gn_offset, float gn_eps, void *out, void *sT);

// with gradients through the state: S_0 = s0 (null = 0), G_T = gsT (null = 0), gs0 = dL/dS_0 (may be null);
// states are fp32 (B,H,64,64) [key][value]
size_t scan_backward_state_workspace_bytes(int64_t B, int64_t T, int64_t C);
hipError_t scan_backward_state(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const float *s0, const void *gy, const float *gsT,
                               void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0, void *workspace);

// --- chunk-parallel MFMA form, bf16 tensors only (wkv6_chunk.hip) ---
hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states,
                         float *dsum = nullptr,    // dsum: see chunk_forward_segments_run
                         bool reverse = false,     // the time axis read back to front (T a multiple of 64, no y)
                         bool counters = true);    // saved_states ends with the per-head counters of the fused gu sum (zeroed here)

// --- block form (wkv6_block_fwd.hip, wkv6_block_bwd.hip): a 64-token chunk as one block of the
// recurrence; bf16 tensors, T a multiple of 64, between half a pair and one pair per compute unit.
// Same arguments and the same saved-state layout as the tile form above, which takes every other case.
// workgroups of a block-form launch (0: the shape is not taken)
int64_t block_grid(int64_t B, int64_t H);
bool block_forward_applies(int64_t B, int64_t T, int64_t H);
hipError_t block_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states, bool counters);

// the block-form forward with the layer's output stage fused in (see chunk_forward_fused / chunk_forward_fused_save):
// y and stats may be null (inference), saved_states null without a backward to follow
hipError_t block_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s0, const int64_t *map, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                               void *out, void *y, float *stats, void *sT, void *saved_states);
bool block_backward_applies(int64_t B, int64_t T, int64_t H);
// workspace: the chunk-start states as a forward pass leaves them, followed by the per-head counters; gu_sum may be null
hipError_t block_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, void *gu_sum,
                          const float *s0 = nullptr, const float *gsT = nullptr, float *gs0 = nullptr);

// --- full-precision chunk form (wkv6_chunk32_fwd.hip, wkv6_chunk32_bwd.hip): fp32 and fp16 tensors on the
// fp32 matrix instructions, chunks of 32 tokens, fp32 states; any T (the last chunk may be short).
bool chunk32_forward_applies(int dtype, int64_t B, int64_t T, int64_t H);
size_t chunk32_saved_bytes(int64_t B, int64_t T, int64_t H);   // one fp32 state per chunk and pair
// saved_states (may be null): receives the chunk-start states for chunk32_backward; y may be null then
hipError_t chunk32_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H,
                           const void *r, const void *k, const void *v, const void *w, const void *u,
                           const void *s0, const int64_t *map, void *y, void *sT, void *saved_states);

// saved_states: what chunk32_forward left (the pair's slice also serves the per-timestep pass of a pair
// whose decay left the chunk form's reach); gu (B, C)
hipError_t chunk32_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                            const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                            void *gr, void *gk, void *gv, void *gw, void *gu, void *saved_states,
                            // gradients through the state ((B,H,64,64) fp32 [key][value]; sT = the forward's final state,
                            // needed with gsT); the saved states come from a forward that started from s0
                            const float *s0 = nullptr, const float *gsT = nullptr, const float *sT = nullptr, float *gs0 = nullptr);

// fp16 tensors on the chunked kernels (training pair only: y and the gradients are fp32).  r, k, w stay
// fp16 (the kernels unpack them exactly); v and gy are consumed as bf16 MFMA operands, so the caller
// keeps bf16 copies of them (convert_to_bf16) next to the saved states.
hipError_t convert_to_bf16(hipStream_t st, int src_dtype, const void *src, void *dst, int64_t n);
hipError_t chunk_forward_save_f16(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                  const void *r, const void *k, const void *v, const void *v_bf16, const void *w, const void *u,
                                  void *y, void *saved_states);

// Few pairs, long sequence: the forward as P time segments side by side (two passes joined by the
// affine map of a segment's state).  chunk_forward_segments = P for the shape (1 = does not apply).
int chunk_forward_segments(int64_t B, int64_t T, int64_t H);
int64_t chunk_forward_segments_remainder(int64_t B, int64_t T, int64_t H);   // tokens behind the P equal segments (single sequence only)
size_t chunk_forward_segments_workspace_bytes(int64_t B, int64_t T, int64_t H);
hipError_t chunk_forward_segments_run(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                                      const void *r, const void *k, const void *v, const void *w, const void *u,
                                      const void *s0, const int64_t *map, void *y, void *sT, void *workspace,
                                      const void *gate = nullptr, const float *gn_scale = nullptr,
                                      const float *gn_offset = nullptr, float gn_eps = 0.f);

// The training pair of a long sequence of few pairs as P time segments side by side.  The saving
// forward leaves, behind the saved chunk states (`extra`), every segment's incoming state and decay
// exponents; the backward chains its reverse state through the same affine maps (two passes each).
struct TrainSegments {
    int P;              // segments per sequence (1: does not apply)
    float *states;      // [B*P][H][64][64] state entering each segment
    float *dsum;        // decay exponents of each segment (as chunk_forward leaves them)
    float *gstates;     // [B*P][H][64][64] gradient arriving at the end of each segment
    void *gu_rows;      // [B*P][C] gu of each segment
    size_t bytes;       // size of the block
};
int chunk_train_segments(int64_t B, int64_t T, int64_t H);
TrainSegments train_segments_layout(int64_t B, int64_t T, int64_t H, void *extra);
// states[(b*P + seg), h]: on entry what each segment builds alone, on exit what enters it (forward: the
// state, from s0 or zero; reverse: the gradient arriving at its end, from `arriving` or zero, and
// `leaving` receives what leaves the first segment, dL/dS_0).
hipError_t segment_chain_forward(hipStream_t st, int P, int64_t B, int64_t H, const float *dsum, float *states, const float *s0);
hipError_t segment_chain_reverse(hipStream_t st, int P, int64_t B, int64_t H, const float *dsum, float *states,
                                 const float *arriving = nullptr, float *leaving = nullptr);
hipError_t chunk_backward_state_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                         const void *r, const void *k, const void *v, const void *w, const void *u,
                                         const float *s0, const void *gy, const float *gsT,
                                         void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0,
                                         void *saved, void *extra);
hipError_t chunk_forward_save_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                       const void *r, const void *k, const void *v, const void *w, const void *u,
                                       void *y, void *saved, void *extra);
hipError_t chunk_backward_saved_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                                         void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum,
                                         void *saved, void *extra);

// forward with the layer's output stage fused in: out = (group_norm_head(y) * gn_scale + gn_offset) * gate
hipError_t chunk_forward_fused(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s0, const int64_t *map, const void *gate, const float *gn_scale,
                               const float *gn_offset, float gn_eps, void *out, void *sT);

// The same for training: also writes y (bf16), the norm's statistics (B,T,H,2: mean, rstd) and the chunk states
hipError_t chunk_forward_fused_save(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                    const void *r, const void *k, const void *v, const void *w, const void *u,
                                    const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                                    void *out, void *y, float *stats, void *saved_states);
// ... of a shape whose training pair runs in time segments (saved / extra as in chunk_forward_save_segments)
hipError_t chunk_forward_fused_save_segments(hipStream_t st, int64_t B, int64_t T, int64_t H,
                                             const void *r, const void *k, const void *v, const void *w, const void *u,
                                             const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                                             void *out, void *y, float *stats, void *saved, void *extra);
// backward of the output stage (wkv6_gn.hip): bf16 tensors, gscale / goffset fp32 (C), zeroed inside
hipError_t gn_gate_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                            const void *gout, const void *y, const float *stats, const void *gate,
                            const float *scale, const float *offset, void *gy, void *ggate, float *gscale, float *goffset);

// input side of the time-mix layer (wkv6_mix.hip): token shift and the five low-rank mixers, bf16 tensors,
// rank R in {32, 64}.  h (B,T,5,R), w2t (5,C,R), bias (5,C) and mix_x (C) fp32.
bool shift_mix_supported(int64_t C, int64_t R);
hipError_t shift_mix_x(hipStream_t st, int64_t B, int64_t T, int64_t C, const void *x, const float *mix_x, void *x_mix);
hipError_t shift_mix_five(hipStream_t st, int64_t B, int64_t T, int64_t C, int64_t R, const void *x, const void *h,
                          const void *w2t, const float *bias, void *const out[5]);
// gcoef: five (B,T,C) planes gcoef_stride elements apart; gp and gxx (B,T,C)
hipError_t shift_mix_five_backward(hipStream_t st, int64_t B, int64_t T, int64_t C, int64_t R, const void *x, const void *h,
                                   const void *w2t, const float *bias, const void *const gout[5], void *gcoef, int64_t gcoef_stride,
                                   void *gp, void *gxx);
// gx (B,T,C), gmix_x (C) fp32, zeroed inside
hipError_t shift_mix_x_backward(hipStream_t st, int64_t B, int64_t T, int64_t C, const void *x, const float *mix_x,
                                const void *gp, const void *gxx, const void *gxm, void *gx, float *gmix_x);

size_t chunk_backward_workspace_bytes(int64_t B, int64_t T, int64_t H);
// bytes of a forward -> backward hand-over buffer: the workspace plus one arrival counter per head
// (zeroed by the saving forward, used by the backward's fused batch sum of gu)
size_t chunk_saved_bytes(int64_t B, int64_t T, int64_t H);
// states_ready: the workspace already holds the chunk-start states (written by a forward pass).
// gu_sum (may be null; needs states_ready and a buffer of chunk_saved_bytes): also write sum_b gu[b].
hipError_t chunk_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, bool states_ready,
                          void *gu_sum, const float *s0 = nullptr, const float *gsT = nullptr, float *gs0 = nullptr,
                          int in_dtype = kBF16, const void *v_orig = nullptr, const void *gy_orig = nullptr);
// s0 / gsT / gs0: gradients through the state, as in scan_backward_state (with states_ready = false)
// in_dtype kF16 (needs states_ready): r, k, w, u fp16, v and gy their bf16 copies, v_orig / gy_orig the
// caller's fp16 v and fp32 gy, gradients fp32

// sum over the batch of (B, C) partials -> (C), both in the output type (for the paths without a fused sum)
hipError_t sum_over_batch(hipStream_t st, int out_dtype, int64_t B, int64_t C, const void *partials, void *sum);

}  // namespace wkv6
