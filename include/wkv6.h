/*
 * wkv6.h -- C ABI of libwkv6_gfx950.so, the MI355X (gfx950) implementation of the WKV6
 * time-mixing operator.  Plain pointers and sizes only; every pointer (state_map and workspace
 * included) is a DEVICE pointer to a row-major contiguous, 16-byte aligned array; all work is
 * enqueued on `stream` (a hipStream_t, may be NULL = default stream) and the calls return
 * without synchronising.  Calls are re-entrant: what the library keeps between calls are per-device
 * caches of things that do not change (compute-unit count, kernel attributes already set, the
 * address of its scratch array); the one exception is wkv6_backward_static, see there.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference tree infiy-quine/STAR-RWKV6).
 *
 * Tensors:  r,k,v,w,y,gy,gr,gk,gv,gw : (B,T,C), channel c = h*N + n, N = C/H (head size);
 *           u : C elements (H,N);  gu : (B,C) per-batch partials (the caller sums over B,
 *           as rwkv_kernel/torch_rwkv_kernel.py:73 and rwkv_kernel/jax_rwkv_kernel.py:166 do);
 *           state s, ys : (n_state|B, H, N, N) indexed [key j][value i]
 *           (rwkv_kernel/ops_rwkv_kernal.py:85-91);  state_map : (B,) int64 on the device.
 *           w is the RAW decay input; the operator applies exp(-exp(w)) itself
 *           (rwkv_kernel/jax_kernel/rwkv_kernels.cu:125).
 * Element types (`dtype` = type of r,k,v,w,u): outputs, gy and states use the "output type":
 *           F32 -> F32, BF16 -> BF16, F16 -> F32 (rwkv_kernel/torch_rwkv_kernel.py:35).
 */
#ifndef WKV6_H_
#define WKV6_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same numbering as `enum ElementType { BF16, F16, F32 }`, rwkv_kernel/jax_kernel/kernels.h:30. */
enum { WKV6_BF16 = 0, WKV6_F16 = 1, WKV6_F32 = 2 };

/* Return codes (the reference's natives return void and assert; this ABI never throws). */
enum {
    WKV6_OK = 0,
    WKV6_ERR_ARG = 1,         /* null pointer, non-positive size, C != H*N, unknown dtype   */
    WKV6_ERR_UNSUPPORTED = 2, /* head size (or path for this head size / dtype) without a kernel   */
    WKV6_ERR_WORKSPACE = 3,   /* workspace missing or smaller than the query function says   */
    WKV6_ERR_LAUNCH = 4       /* the HIP runtime refused a launch (see wkv6_last_hip_error)   */
};

/* Algorithm selector for the *_ex entry points. */
enum {
    WKV6_ALGO_AUTO = 0,  /* library picks.  bf16 tensors with T >= 32: chunked bf16-MFMA path.  fp32 and
                            fp16 tensors with T >= 64: the full-precision chunk form (every product on
                            the fp32 matrix instructions, chunks of 32 tokens, fp32 accuracy: y within
                            1e-4, gradients within 1e-3 relative, the same y with and without a
                            gradient; its training pair saves one fp32 state per chunk; gradients
                            through the state included).  Everything else: the per-timestep
                            kernels                                                             */
    WKV6_ALGO_SCAN = 1,  /* per-timestep fp32 recurrence, state in VGPRs                       */
    WKV6_ALGO_CHUNK = 2  /* chunk-parallel form.  bf16 tensors: bf16 MFMA for the dense intra-chunk
                            products in every call.  fp32 tensors: the full-precision chunk form, as
                            under AUTO.  fp16 tensors (fp32 outputs): the training pair
                            wkv6_forward_save / wkv6_backward_saved* runs on the bf16-MFMA kernels
                            (r, k, w unpacked exactly; v, gy reach the MFMAs as bf16 copies kept in
                            the saved block); calls without a gradient run the full-precision chunk
                            form.  ACCURACY: for the fp16 training pair this is an explicit trade --
                            the fp32-typed y and gradients then carry bf16 operand precision
                            (relative error up to 1e-2, against 1e-4 under AUTO), and differ by
                            that much from what wkv6_forward returns for the same inputs.  In
                            either chunk form a (batch, head) pair whose decay goes beyond what the
                            operand scaling can hold is redone with the exact per-timestep code
                            inside the same launch                                             */
};

const char *wkv6_status_string(int status);
int wkv6_version(void);
/* Head sizes compiled into the library: returns 1 if N is supported.  64: every entry point.  Every other multiple of
 * 4 up to 128 (the reference builds for any multiple of 4, rwkv_kernel/torch_rwkv_kernel.py:13; its scripts run 8
 * and 32): the
 * plain calls -- wkv6_forward*, wkv6_forward_with_state*, wkv6_backward*, wkv6_backward_with_state, the
 * training pair (which then saves nothing: wkv6_saved_bytes = 0) and the XLA targets -- on per-timestep fp32
 * kernels with one thread per channel, states (B, H, N, N); WKV6_ALGO_CHUNK, the fused stages and
 * wkv6_backward_static answer WKV6_ERR_UNSUPPORTED for them. */
int wkv6_supports_head_size(int64_t N);

/* Stateless forward.
 * Replaces forward_{bf16,fp16,fp32}(B,T,C,H,r,k,v,w,u,y), rwkv_kernel/torch_kernel/wkv6_op.cpp:22-30,
 * i.e. cuda_forward<>, rwkv_kernel/torch_kernel/wkv6_cuda.cu:323-329 (kernel_forward). */
int wkv6_forward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                 const void *r, const void *k, const void *v, const void *w, const void *u,
                 void *y);

/* Forward with optional initial state and final-state output.
 * Replaces forward_with_state_{bf16,fp16,fp32}(B,T,C,H,S,map,r,k,v,w,u,s,y,ys),
 * rwkv_kernel/torch_kernel/wkv6_op.cpp:44-52 (kernel_forward_state,
 * rwkv_kernel/jax_kernel/rwkv_kernels.cu:165-190).  has_init_state==0: s and state_map ignored,
 * zero initial state.  has_init_state!=0: S_0[b] = s[state_map[b]] (state_map NULL = identity);
 * state_map values must lie in [0, rows of s) -- validated by the caller on the host.
 * s and ys are in the output type.  ys may alias s only when state_map is the identity. */
int wkv6_forward_with_state(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                            int has_init_state, const int64_t *state_map,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const void *s, void *y, void *ys);

/* Same, with the state element type chosen separately (WKV6_F32 keeps a decode loop's carried
 * state in fp32 while the activations stay bf16).  No counterpart in the reference, whose state
 * type is always the output type (rwkv_kernel/torch_rwkv_kernel.py:126-131). */
int wkv6_forward_with_state_ex(void *stream, int dtype, int state_dtype, int algo,
                               int64_t B, int64_t T, int64_t C, int64_t H,
                               int has_init_state, const int64_t *state_map,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s, void *y, void *ys,
                               void *workspace, size_t workspace_bytes);
/* Optional workspace of wkv6_forward_ex / wkv6_forward_with_state_ex (0 = none useful).  Where it is
 * non-zero -- a long bf16 sequence with so few (batch, head) pairs that most of the chip would idle --
 * passing that many bytes lets the forward run as time segments side by side (same results to
 * rounding); without it the call works as always.  Batches need T to divide into equal segments
 * of whole 64-token chunks; a single sequence (B = 1) may have any length if its final state is
 * fp32 or not asked for. */
size_t wkv6_forward_workspace_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);

/* Forward (inference) with the layer's output stage fused in; y itself is not written:
 *     out[b,t,h,:] = (layer_norm(y[b,t,h,:], gn_eps) * gn_scale[h,:] + gn_offset[h,:]) * gate[b,t,h,:]
 * i.e. what the caller of the operator does next in the reference model: the per-head group
 * normalisation with learned scale and offset and the gate, rwkv6_model.py:94-99 (GroupNorm.call,
 * mean and variance over one head's channels) and :158-160 (TimeMix.call: x = group_norm(x) * g).
 * No counterpart in the reference's native code, which leaves these to framework kernels (one more
 * write and two more reads of a (B,T,C) tensor per layer).  bf16 tensors only (WKV6_ERR_UNSUPPORTED
 * otherwise); gn_scale, gn_offset: (H, 64) fp32 in device memory; gate, out: (B,T,C) in `dtype`;
 * state arguments as in wkv6_forward_with_state_ex (ys may be NULL).  No gradient. */
int wkv6_forward_gn_gate(void *stream, int dtype, int state_dtype,
                         int64_t B, int64_t T, int64_t C, int64_t H,
                         int has_init_state, const int64_t *state_map,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                         void *out, void *ys);
/* Same with the optional workspace of wkv6_forward_workspace_bytes(dtype, WKV6_ALGO_CHUNK, ...): a long
 * sequence of few (batch, head) pairs then runs as time segments side by side.  No counterpart in the
 * reference. */
int wkv6_forward_gn_gate_ex(void *stream, int dtype, int state_dtype,
                            int64_t B, int64_t T, int64_t C, int64_t H,
                            int has_init_state, const int64_t *state_map,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const void *s, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                            void *out, void *ys, void *workspace, size_t workspace_bytes);

/* The same output stage for TRAINING (no counterpart in the reference, which leaves the group norm and
 * the gate -- rwkv6_model.py:94-99,158-160 -- and their gradients to framework kernels):
 *
 * wkv6_forward_gn_gate_save: zero initial state; writes `out` as above and, for the backward, y
 * (B,T,C) bf16, the norm's statistics `stats` (B,T,H,2) fp32 = (mean, 1/sqrt(var + gn_eps)) of y over
 * each head's channels, and the chunk states into `saved` (wkv6_saved_bytes(dtype, WKV6_ALGO_CHUNK, ...)
 * bytes, as for wkv6_forward_save).  bf16 tensors only.  Where the training pair runs in time segments (few
 * pairs, long sequence) the output stage is part of the segments' second pass.
 *
 * wkv6_gn_gate_backward: given gout = dL/dout, writes gy = dL/dy (feed it to wkv6_backward_saved* with
 * the same `saved`), ggate = dL/dgate (both (B,T,C) bf16) and gscale, goffset = dL/dgn_scale,
 * dL/dgn_offset ((H,64) fp32, summed over batch and time; zeroed by the call). */
int wkv6_forward_gn_gate_save_supported(int dtype, int64_t B, int64_t T, int64_t C, int64_t H);   /* 1: this shape is taken */
int wkv6_forward_gn_gate_save(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                              const void *r, const void *k, const void *v, const void *w, const void *u,
                              const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                              void *out, void *y, float *stats, void *saved, size_t saved_bytes);
int wkv6_gn_gate_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                          const void *gout, const void *y, const float *stats, const void *gate,
                          const float *gn_scale, const float *gn_offset,
                          void *gy, void *ggate, float *gscale, float *goffset);

/* The INPUT side of the layer around the operator (no counterpart in the reference, which leaves it
 * to framework kernels): the token shift and the five low-rank mixers of rwkv6_model.py:134-146 that
 * turn the layer input x into the inputs xr, xk, xv, xw, xg of the projections producing r, k, v, w
 * and the gate.  With xx = (previous token, zero before the first) - x  (TimeShift, :40-43):
 *
 *   wkv6_shift_mix_x:     x_mix = x + xx * mix_x                                  (:136)
 *   (caller)              h[:, :, s, :] = tanh(x_mix A_s^T), s = r,k,v,w,g        (DecomposerDense.dense_a, :20)
 *   wkv6_shift_mix_five:  x_s = x + xx * (h_s W_s^T + bias_s)                     (dense_b :21, :141-145)
 *
 * The rank-R product h_s W_s^T runs on the matrix cores inside the kernel that writes the five
 * outputs, so the five (B,T,C) coefficient tensors are never stored.  bf16 tensors; C a multiple
 * of 64; R (decomposer_size) 32 or 64 -- wkv6_shift_mix_supported says whether a shape is taken,
 * WKV6_ERR_UNSUPPORTED otherwise.  x, x_mix, x_s and their gradients (B,T,C); h (B,T,5,R);
 * w2t (5,C,R): each mixer's dense_b weight as (out, in); bias (5,C) and mix_x (C) fp32.
 *
 * Backward, in the order the chain rule needs it:
 *   wkv6_shift_mix_five_backward: from the gradients gx_s of the five outputs writes
 *       gcoef = gx_s * xx, five (B,T,C) planes gcoef_stride elements apart (at least B*T*C, a
 *       multiple of 8)  -- the caller's GEMMs turn it into the gradients of h
 *       (gcoef_s W_s), of W_s (gcoef_s^T h_s) and of bias_s (sum over tokens) --,
 *       gxx = sum_s gx_s * coef_s and gp = sum_s gx_s - gxx  (both (B,T,C)).
 *   (caller) gh -> through tanh and A -> gxm = dL/dx_mix (B,T,C)
 *   wkv6_shift_mix_x_backward: gx = gp + gxm (1 - mix_x) + z[t+1] with z = gxx + gxm mix_x
 *       (nothing from beyond a sequence's last token), gmix_x (C) fp32 = sum over tokens of gxm * xx
 *       (zeroed by the call).  gp and gxx may both be NULL (zero): the backward of x_mix alone, e.g. for
 *       the channel-mix layer's two fixed token-shift mixes (rwkv6_model.py:57-60). */
int wkv6_shift_mix_supported(int dtype, int64_t C, int64_t R);
int wkv6_shift_mix_x(void *stream, int dtype, int64_t B, int64_t T, int64_t C,
                     const void *x, const float *mix_x, void *x_mix);
int wkv6_shift_mix_five(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t R,
                        const void *x, const void *h, const void *w2t, const float *bias,
                        void *xr, void *xk, void *xv, void *xw, void *xg);
int wkv6_shift_mix_five_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t R,
                                 const void *x, const void *h, const void *w2t, const float *bias,
                                 const void *gxr, const void *gxk, const void *gxv, const void *gxw, const void *gxg,
                                 void *gcoef, int64_t gcoef_stride, void *gp, void *gxx);
int wkv6_shift_mix_x_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C,
                              const void *x, const float *mix_x, const void *gp, const void *gxx, const void *gxm,
                              void *gx, float *gmix_x);

/* Backward of the stateless forward: gr,gk,gv,gw (B,T,C) and gu (B,C), all in the output type.
 * Replaces backward_{bf16,fp16,fp32}(B,T,C,H,r,k,v,w,u,gy,gr,gk,gv,gw,gu),
 * rwkv_kernel/torch_kernel/wkv6_op.cpp:33-41 (kernel_backward_101/102/103/201,
 * rwkv_kernel/jax_kernel/rwkv_kernels.cu:205-407, launched by HostApplyGradient :436-444).
 * `workspace` is device memory of at least wkv6_backward_workspace_bytes(...) bytes owned by the
 * caller; its contents on entry and exit are meaningless.  (What it holds depends on the kernels the
 * shape takes -- 4 bytes per element of r on the per-timestep kernels and the bf16 chunk forms, one
 * fp32 64x64 state per 32 tokens and head = 8 bytes per element of r on the full-precision chunk form of
 * fp32 / fp16 tensors -- so size it with the query, not by hand.) */
int wkv6_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                  const void *r, const void *k, const void *v, const void *w, const void *u,
                  const void *gy,
                  void *gr, void *gk, void *gv, void *gw, void *gu,
                  void *workspace, size_t workspace_bytes);
size_t wkv6_backward_workspace_bytes(int dtype, int64_t B, int64_t T, int64_t C, int64_t H);

/* wkv6_backward without a workspace argument and without any allocation: the workspace is a
 * fixed array in device memory that belongs to the library (WKV6_STATIC_SCRATCH_BYTES, present on
 * every GPU the library is used on from the first such call until the process ends).  No
 * counterpart in the reference; it is for callers that cannot allocate device memory at the
 * point of the call -- code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc -- and neither the library nor anything it calls allocates or frees memory here (the
 * first call on a device looks the array's address up once).  Shapes whose
 * wkv6_backward_workspace_bytes() exceeds WKV6_STATIC_SCRATCH_BYTES run on the per-timestep kernels
 * if their workspace (4 bytes per element of r) fits, and are refused with WKV6_ERR_WORKSPACE
 * otherwise (the benchmark shape B=8 T=1024 C=2048 needs exactly the array's size, as bf16 on the
 * chunked kernels and as fp32 on the per-timestep ones).  All calls
 * on one GPU share the one array: two calls whose kernels overlap in time on the same GPU
 * (different streams, different host threads) race -- serialise them.  Same results as
 * wkv6_backward. */
#define WKV6_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int wkv6_backward_static(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu);

/* Same two calls with the algorithm forced (tests and benchmarks compare the two paths). */
int wkv6_forward_ex(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                    const void *r, const void *k, const void *v, const void *w, const void *u,
                    void *y, void *workspace, size_t workspace_bytes);
int wkv6_backward_ex(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                     const void *r, const void *k, const void *v, const void *w, const void *u,
                     const void *gy,
                     void *gr, void *gk, void *gv, void *gw, void *gu,
                     void *workspace, size_t workspace_bytes);
size_t wkv6_backward_workspace_bytes_ex(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);

/* Training pair: a forward that also saves what the backward can reuse (bf16 tensors on the chunked
 * kernels: the state at every 64-token chunk start, as bf16; fp32 and fp16 tensors on the full-precision
 * chunk form: the fp32 state at every 32-token chunk start), and the backward that consumes it and therefore
 * skips its own forward state sweep.  `saved` is caller-owned device memory of wkv6_saved_bytes()
 * bytes (0 = this path saves nothing; pass NULL), must be left untouched between the two calls,
 * and serves the backward as its workspace too.  A long sequence (T >= 1024) of so few (batch, head)
 * pairs that they fill at most half of the compute units runs as 2, 4, 8 or 16 time segments side by
 * side in both calls (same results to rounding); wkv6_saved_bytes() includes what that keeps.
 * No counterpart in the reference, whose backward
 * recomputes everything from the inputs (rwkv_kernel/torch_rwkv_kernel.py:33 saves only r,k,v,w,u). */
size_t wkv6_saved_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);
int wkv6_forward_save(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                      const void *r, const void *k, const void *v, const void *w, const void *u,
                      void *y, void *saved, size_t saved_bytes);
int wkv6_backward_saved(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                        const void *r, const void *k, const void *v, const void *w, const void *u,
                        const void *gy,
                        void *gr, void *gk, void *gv, void *gw, void *gu,
                        void *saved, size_t saved_bytes);

/* wkv6_backward_saved with the batch sum of gu fused in: gu (B,C) still receives the per-batch
 * partials, gu_sum (C elements, output type) their sum over the batch, added up in fp32 from the
 * stored partials -- the value `gu = torch.sum(gu, 0)` gives the caller in
 * rwkv_kernel/torch_rwkv_kernel.py:73 (rwkv_kernel/jax_rwkv_kernel.py:166), without the extra
 * kernel.  `saved` must come from wkv6_forward_save of the same shape (it carries per-head arrival
 * counters, which the call leaves ready for another backward on the same buffer). */
int wkv6_backward_saved_sum(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const void *gy,
                            void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum,
                            void *saved, size_t saved_bytes);

/* Backward with gradients through the state (no counterpart in the reference, whose backward is
 * defined for the stateless call only, rwkv_kernel/torch_rwkv_kernel.py:100-168; it is what carrying
 * the state across calls, rwkv_kernel/__init__.py:14-38, needs for truncated back-propagation over
 * pieces of a longer sequence).  Gradient of  sum(y*gy) + sum(S_T*gsT)  for the forward started from
 * S_0 = s0:  s0, gsT, gs0 are fp32 (B,H,64,64) in [key][value] order; s0 NULL = zero initial state,
 * gsT NULL = no gradient arrives at the final state, gs0 NULL = dL/dS_0 not wanted.  With a state
 * the first / last decay do receive a gradient (gw[:,0], gw[:,T-1] are not forced to zero).  All
 * three NULL gives wkv6_backward_ex.  gu is (B,C) per-batch partials as in wkv6_backward. */
size_t wkv6_backward_with_state_workspace_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);
int wkv6_backward_with_state(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                             const void *r, const void *k, const void *v, const void *w, const void *u,
                             const float *s0, const void *gy, const float *gsT,
                             void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0,
                             void *workspace, size_t workspace_bytes);

/* ---- XLA custom-call surface (replaces the pybind module `gpu_ops`,
 * rwkv_kernel/jax_kernel/gpu_ops.cpp:20-43) ---------------------------------------------- */

/* 28-byte opaque descriptor, same field order as WKVDescriptor, rwkv_kernel/jax_kernel/kernels.h:32-42. */
typedef struct wkv6_descriptor {
    int32_t B, T, C, H;
    uint8_t S;        /* has initial state */
    uint8_t pad_[3];
    int32_t x_type;   /* WKV6_BF16 | WKV6_F16 | WKV6_F32 */
    int32_t y_type;
} wkv6_descriptor;

/* Replaces create_rwkv_descriptor (gpu_ops.cpp:33-36): fills out[0..28), returns 28. */
size_t wkv6_create_descriptor(int B, int T, int C, int H, int S, int x_type, int y_type, void *out);

/* XLA status-less custom-call targets, signature void(stream, buffers, opaque, opaque_len)
 * (rwkv_kernel/jax_kernel/kernels.h:44-53).  Buffer order = operands then results:
 *   wkv_forward            [r,k,v,w,u | y]                                (rwkv_kernels.cu:458-462)
 *   wkv_backward           [r,k,v,w,u,gy | gr,gk,gv,gw,gu(B,C), workspace] (rwkv_kernels.cu:500-506,
 *                          plus one trailing scratch result of wkv6_backward_workspace_bytes bytes)
 *   wkv_forward_with_state S=1: [map,r,k,v,w,u,s | y,ys]   S=0: [r,k,v,w,u | y,ys]   (:474-488)
 * A wrong opaque_len makes the call a no-op and records WKV6_ERR_ARG (wkv6_last_status);
 * nothing is thrown across the boundary (the reference throws, kernel_helpers.h:56-58). */
void wkv_forward(void *stream, void **buffers, const char *opaque, size_t opaque_len);
void wkv_backward(void *stream, void **buffers, const char *opaque, size_t opaque_len);
void wkv_forward_with_state(void *stream, void **buffers, const char *opaque, size_t opaque_len);
/* Two more targets, for the forward and backward rules of the custom_vjp (rwkv_kernel/jax_rwkv_kernel.py:148-170
 * registers wkv_forward and wkv_backward there): the training pair wkv6_forward_save / wkv6_backward_saved_sum
 * under WKV6_ALGO_AUTO, for shapes with wkv6_saved_bytes(x_type, WKV6_ALGO_AUTO, ...) = n > 0 (otherwise
 * WKV6_ERR_UNSUPPORTED is recorded and nothing runs).  No counterpart in the reference, whose backward
 * recomputes everything from the inputs.
 *   wkv_forward_save    [r,k,v,w,u | y, saved(n bytes)]
 *   wkv_backward_saved  [r,k,v,w,u,gy,saved | gr,gk,gv,gw,gu(B,C), saved_out(n bytes), gu_sum(C)]
 * The backward uses parts of the block as scratch, so the caller declares saved_out as an alias of the
 * operand saved (output_operand_aliases / input_output_aliases={6: 5}); given two different buffers the
 * target copies the operand into the result first and leaves the operand alone. */
void wkv_forward_save(void *stream, void **buffers, const char *opaque, size_t opaque_len);
void wkv_backward_saved(void *stream, void **buffers, const char *opaque, size_t opaque_len);
/* Status of the calling thread's most recent custom-call target invocation. */
int wkv6_last_status(void);
/* hipError_t value of the calling thread's most recent failed launch (0 if none). */
int wkv6_last_hip_error(void);

#ifdef __cplusplus
}
#endif
#endif /* WKV6_H_ */
