// C ABI of libwkv6_gfx950.so: argument validation, algorithm choice, launch.  See include/wkv6.h.
#include "wkv6.h"
#include "wkv6_kernels.h"

#include <string.h>

#include <atomic>

// Workspace of wkv6_backward_static: device memory the library owns, one copy per GPU.  In host
// code the name below is only a handle for hipGetSymbolAddress; the address that kernels, copies and
// memsets take is looked up per device (static_scratch()).
static __device__ __align__(256) unsigned char scratch[WKV6_STATIC_SCRATCH_BYTES];

namespace {

// Device address of `scratch` on the current device (null on failure, *err says why); looked up on
// the first call per device.
void *static_scratch(hipError_t *err) {
    static std::atomic<void *> ptr[64];
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= 64) { *err = hipErrorInvalidDevice; return nullptr; }
    void *p = ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (*err != hipSuccess) return nullptr;
        ptr[dev].store(p, std::memory_order_release);
    }
    return p;
}

// Shapes the chunked MFMA kernels take; everything else runs the per-timestep kernels.
// (the chunked kernels index one batch row with 32-bit element offsets)
bool chunk_possible(int dtype, int64_t T, int64_t C) { return dtype == WKV6_BF16 && T * C < (1LL << 31); }
bool chunk_eligible(int dtype, int64_t T, int64_t C) { return chunk_possible(dtype, T, C) && T >= 32; }

// The training pair (wkv6_forward_save / wkv6_backward_saved*) can also run fp16 tensors on the chunked
// kernels: r, k, w are unpacked exactly, v and gy go through bf16 copies kept behind the saved states.
// That gives fp32-typed outputs of bf16 operand precision (1e-2 class), which differ from what the
// exact per-timestep kernels return for the same fp16 inputs (every call without a gradient takes
// those): only on request (WKV6_ALGO_CHUNK), never under WKV6_ALGO_AUTO.
bool train_chunk(int dtype, int algo, int64_t T, int64_t C) {
    if (dtype != WKV6_BF16 && dtype != WKV6_F16) return false;
    // (the kernels address a (b, h) pair's rows with 32-bit byte offsets; fp16 tensors have 4-byte outputs)
    if (T * C >= (dtype == WKV6_F16 ? 1LL << 30 : 1LL << 31)) return false;
    return algo == WKV6_ALGO_CHUNK || (algo == WKV6_ALGO_AUTO && dtype == WKV6_BF16 && T >= 32);
}

// fp32 tensors, and fp16 tensors unless their training pair asks for the bf16-operand kernels, train on the
// full-precision chunk form; the per-timestep kernels on request (WKV6_ALGO_SCAN) and for short sequences.
bool train_chunk32(int dtype, int algo, int64_t B, int64_t T, int64_t H) {
    if (algo == WKV6_ALGO_SCAN || (dtype == WKV6_F16 && algo == WKV6_ALGO_CHUNK)) return false;
    return wkv6::chunk32_forward_applies(dtype, B, T, H);
}

thread_local int g_last_status = WKV6_OK;
thread_local int g_last_hip_error = 0;

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// WKV6_OK: head size 64, every entry point.  kSmallHead: another head size that is a multiple of 4, up to 128 (otherwise valid), which the plain
// calls (forward, forward with state, backward, backward with state, the training pair without saved states)
// serve with the kernels of wkv6_generic.hip and every other entry point refuses as unsupported.
constexpr int kSmallHead = -1;
int check_shape_any(int dtype, int64_t B, int64_t T, int64_t C, int64_t H) {
    if (dtype != WKV6_BF16 && dtype != WKV6_F16 && dtype != WKV6_F32) return WKV6_ERR_ARG;
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0 || C % H != 0) return WKV6_ERR_ARG;
    if (B * H > 0x7fffffffLL || T > 0x7fffffffLL) return WKV6_ERR_ARG;
    if (C / H == 64) return WKV6_OK;
    if (wkv6::generic_head_size(C / H)) return B <= 65535 && B * T * C < (1LL << 40) ? kSmallHead : WKV6_ERR_UNSUPPORTED;
    return WKV6_ERR_UNSUPPORTED;
}
int check_shape(int dtype, int64_t B, int64_t T, int64_t C, int64_t H) {
    const int rc = check_shape_any(dtype, B, T, C, H);
    return rc == kSmallHead ? WKV6_ERR_UNSUPPORTED : rc;
}

int out_type(int dtype) { return dtype == WKV6_BF16 ? WKV6_BF16 : WKV6_F32; }

int finish(hipError_t e) {
    if (e != hipSuccess) { g_last_hip_error = (int)e; return WKV6_ERR_LAUNCH; }
    return WKV6_OK;
}

}  // namespace

extern "C" {

const char *wkv6_status_string(int s) {
    switch (s) {
    case WKV6_OK: return "ok";
    case WKV6_ERR_ARG: return "invalid argument (null/misaligned pointer, bad size or dtype)";
    case WKV6_ERR_UNSUPPORTED: return "unsupported: head size (64 everywhere; other multiples of 4 up to 128 in the plain calls) or a path this dtype / shape has no kernel for";
    case WKV6_ERR_WORKSPACE: return "workspace missing or too small";
    case WKV6_ERR_LAUNCH: return "HIP launch failed";
    default: return "unknown status";
    }
}

int wkv6_version(void) { return 100; }
int wkv6_supports_head_size(int64_t N) { return N == 64 || wkv6::generic_head_size(N); }
int wkv6_last_status(void) { return g_last_status; }
int wkv6_last_hip_error(void) { return g_last_hip_error; }

size_t wkv6_forward_workspace_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    if (check_shape(dtype, B, T, C, H) != WKV6_OK) return 0;
    const bool chunk = (algo == WKV6_ALGO_CHUNK && chunk_possible(dtype, T, C)) ||
                       (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    // optional: with it, a long sequence of few (batch, head) pairs runs as time segments side by side
    return chunk ? wkv6::chunk_forward_segments_workspace_bytes(B, T, H) : 0;
}

static int forward_impl(void *stream, int dtype, int state_dtype, int algo,
                        int64_t B, int64_t T, int64_t C, int64_t H,
                        int has_init_state, const int64_t *state_map,
                        const void *r, const void *k, const void *v, const void *w, const void *u,
                        const void *s, void *y, void *ys, void *saved,
                        void *workspace = nullptr, size_t workspace_bytes = 0) {
    int rc = check_shape_any(dtype, B, T, C, H);
    if (rc != WKV6_OK && rc != kSmallHead) return rc;
    if (!r || !k || !v || !w || !u || !y) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(y)) return WKV6_ERR_ARG;
    if (has_init_state && !s) return WKV6_ERR_ARG;
    if (state_dtype != out_type(dtype) && state_dtype != WKV6_F32) return WKV6_ERR_ARG;
    if (algo < WKV6_ALGO_AUTO || algo > WKV6_ALGO_CHUNK) return WKV6_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const void *s_in = has_init_state ? s : nullptr;
    const int64_t *map_in = has_init_state ? state_map : nullptr;
    if (rc == kSmallHead) {
        if (algo == WKV6_ALGO_CHUNK) return WKV6_ERR_UNSUPPORTED;
        return finish(wkv6::generic_forward(st, dtype, state_dtype, B, T, H, C / H, r, k, v, w, u, s_in, map_in, y, ys));
    }
    // fp32 and fp16 tensors: the full-precision chunk form, unless the per-timestep kernels are asked for
    if (algo != WKV6_ALGO_SCAN && wkv6::chunk32_forward_applies(dtype, B, T, H))
        return finish(wkv6::chunk32_forward(st, dtype, state_dtype, B, T, H, r, k, v, w, u, s_in, map_in, y, ys, saved));
    if (algo == WKV6_ALGO_CHUNK && !chunk_possible(dtype, T, C)) return WKV6_ERR_UNSUPPORTED;
    const bool chunk = algo == WKV6_ALGO_CHUNK ||
                       (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    if (!chunk)
        return finish(wkv6::scan_forward(st, dtype, state_dtype, B, T, H, r, k, v, w, u, s_in, map_in, y, ys));
    if (!saved && workspace && aligned16(workspace)) {
        const size_t need = wkv6::chunk_forward_segments_workspace_bytes(B, T, H);
        // (tokens left over behind the equal segments are run from an fp32 state: possible when the
        // final state is fp32 or not wanted)
        const bool remainder_ok = wkv6::chunk_forward_segments_remainder(B, T, H) == 0 || state_dtype == WKV6_F32 || !ys;
        if (need > 0 && workspace_bytes >= need && remainder_ok)
            return finish(wkv6::chunk_forward_segments_run(st, state_dtype, B, T, H, r, k, v, w, u, s_in, map_in, y, ys, workspace));
    }
    return finish(wkv6::chunk_forward(st, state_dtype, B, T, H, r, k, v, w, u, s_in, map_in, y, ys, saved));
}

int wkv6_forward_with_state_ex(void *stream, int dtype, int state_dtype, int algo,
                               int64_t B, int64_t T, int64_t C, int64_t H,
                               int has_init_state, const int64_t *state_map,
                               const void *r, const void *k, const void *v, const void *w, const void *u,
                               const void *s, void *y, void *ys, void *workspace, size_t workspace_bytes) {
    return forward_impl(stream, dtype, state_dtype, algo, B, T, C, H, has_init_state, state_map, r, k, v, w, u, s, y, ys,
                        nullptr, workspace, workspace_bytes);
}

int wkv6_forward_gn_gate(void *stream, int dtype, int state_dtype,
                         int64_t B, int64_t T, int64_t C, int64_t H,
                         int has_init_state, const int64_t *state_map,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                         void *out, void *ys) {
    return wkv6_forward_gn_gate_ex(stream, dtype, state_dtype, B, T, C, H, has_init_state, state_map, r, k, v, w, u, s,
                                   gate, gn_scale, gn_offset, gn_eps, out, ys, nullptr, 0);
}

int wkv6_forward_gn_gate_ex(void *stream, int dtype, int state_dtype,
                            int64_t B, int64_t T, int64_t C, int64_t H,
                            int has_init_state, const int64_t *state_map,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const void *s, const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                            void *out, void *ys, void *workspace, size_t workspace_bytes) {
    int rc = check_shape(dtype, B, T, C, H);
    if (rc != WKV6_OK) return rc;
    if (!r || !k || !v || !w || !u || !gate || !gn_scale || !gn_offset || !out) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gate) || !aligned16(out)) return WKV6_ERR_ARG;
    if (has_init_state && !s) return WKV6_ERR_ARG;
    if (!(gn_eps >= 0.f)) return WKV6_ERR_ARG;
    if (state_dtype != out_type(dtype) && state_dtype != WKV6_F32) return WKV6_ERR_ARG;
    if (!chunk_possible(dtype, T, C)) return WKV6_ERR_UNSUPPORTED;   // bf16 tensors only
    if (T == 1)   // a decode step: the single-timestep kernel
        return finish(wkv6::step_forward_fused((hipStream_t)stream, state_dtype, B, H, r, k, v, w, u,
                                               has_init_state ? s : nullptr, has_init_state ? state_map : nullptr,
                                               gate, gn_scale, gn_offset, gn_eps, out, ys));
    if (workspace && aligned16(workspace)) {   // optional: few pairs, long sequence -> time segments side by side
        const size_t need = wkv6::chunk_forward_segments_workspace_bytes(B, T, H);
        const bool remainder_ok = wkv6::chunk_forward_segments_remainder(B, T, H) == 0 || state_dtype == WKV6_F32 || !ys;
        if (need > 0 && workspace_bytes >= need && remainder_ok)
            return finish(wkv6::chunk_forward_segments_run((hipStream_t)stream, state_dtype, B, T, H, r, k, v, w, u,
                                                           has_init_state ? s : nullptr, has_init_state ? state_map : nullptr,
                                                           out, ys, workspace, gate, gn_scale, gn_offset, gn_eps));
    }
    return finish(wkv6::chunk_forward_fused((hipStream_t)stream, state_dtype, B, T, H, r, k, v, w, u,
                                            has_init_state ? s : nullptr, has_init_state ? state_map : nullptr,
                                            gate, gn_scale, gn_offset, gn_eps, out, ys));
}

static int train_segments(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);
static size_t saved_base_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H);

int wkv6_forward_gn_gate_save_supported(int dtype, int64_t B, int64_t T, int64_t C, int64_t H) {
    return check_shape(dtype, B, T, C, H) == WKV6_OK && dtype == WKV6_BF16 && chunk_possible(dtype, T, C);
}

int wkv6_forward_gn_gate_save(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                              const void *r, const void *k, const void *v, const void *w, const void *u,
                              const void *gate, const float *gn_scale, const float *gn_offset, float gn_eps,
                              void *out, void *y, float *stats, void *saved, size_t saved_bytes) {
    int rc = check_shape(dtype, B, T, C, H);
    if (rc != WKV6_OK) return rc;
    if (dtype != WKV6_BF16 || !chunk_possible(dtype, T, C)) return WKV6_ERR_UNSUPPORTED;
    if (!r || !k || !v || !w || !u || !gate || !gn_scale || !gn_offset || !out || !y || !stats) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gate) || !aligned16(out) || !aligned16(y) ||
        !aligned16(stats) || !aligned16(gn_scale) || !aligned16(gn_offset)) return WKV6_ERR_ARG;
    if (!(gn_eps >= 0.f)) return WKV6_ERR_ARG;
    const size_t need = wkv6_saved_bytes(dtype, WKV6_ALGO_CHUNK, B, T, C, H);
    if (!saved || saved_bytes < need || !aligned16(saved)) return WKV6_ERR_WORKSPACE;
    const int P = train_segments(dtype, WKV6_ALGO_CHUNK, B, T, C, H);
    if (P > 1) {   // few pairs, long sequence: time segments side by side, the output stage in their second pass
        char *extra = reinterpret_cast<char *>(saved) + saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H);
        return finish(wkv6::chunk_forward_fused_save_segments((hipStream_t)stream, B, T, H, r, k, v, w, u, gate, gn_scale, gn_offset,
                                                              gn_eps, out, y, stats, saved, extra));
    }
    return finish(wkv6::chunk_forward_fused_save((hipStream_t)stream, B, T, H, r, k, v, w, u, gate, gn_scale, gn_offset, gn_eps,
                                                 out, y, stats, saved));
}

int wkv6_gn_gate_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                          const void *gout, const void *y, const float *stats, const void *gate,
                          const float *gn_scale, const float *gn_offset,
                          void *gy, void *ggate, float *gscale, float *goffset) {
    int rc = check_shape(dtype, B, T, C, H);
    if (rc != WKV6_OK) return rc;
    if (dtype != WKV6_BF16) return WKV6_ERR_UNSUPPORTED;
    if (!gout || !y || !stats || !gate || !gn_scale || !gn_offset || !gy || !ggate || !gscale || !goffset) return WKV6_ERR_ARG;
    if (!aligned16(gout) || !aligned16(y) || !aligned16(stats) || !aligned16(gate) || !aligned16(gn_scale) || !aligned16(gn_offset) ||
        !aligned16(gy) || !aligned16(ggate) || !aligned16(gscale) || !aligned16(goffset)) return WKV6_ERR_ARG;
    return finish(wkv6::gn_gate_backward((hipStream_t)stream, B, T, H, gout, y, stats, gate, gn_scale, gn_offset, gy, ggate, gscale, goffset));
}

static int check_mix(int dtype, int64_t B, int64_t T, int64_t C, int64_t R) {
    if (B <= 0 || T <= 0 || C <= 0 || R <= 0) return WKV6_ERR_ARG;
    if (dtype != WKV6_BF16 || !wkv6::shift_mix_supported(C, R)) return WKV6_ERR_UNSUPPORTED;
    if (B * T > ((int64_t)1 << 31) / 256 * 64) return WKV6_ERR_UNSUPPORTED;   // the launch grids are 32-bit
    return WKV6_OK;
}

int wkv6_shift_mix_supported(int dtype, int64_t C, int64_t R) {
    return dtype == WKV6_BF16 && wkv6::shift_mix_supported(C, R);
}

int wkv6_shift_mix_x(void *stream, int dtype, int64_t B, int64_t T, int64_t C,
                     const void *x, const float *mix_x, void *x_mix) {
    const int rc = check_mix(dtype, B, T, C, 32);
    if (rc != WKV6_OK) return rc;
    if (!x || !mix_x || !x_mix) return WKV6_ERR_ARG;
    if (!aligned16(x) || !aligned16(mix_x) || !aligned16(x_mix)) return WKV6_ERR_ARG;
    return finish(wkv6::shift_mix_x((hipStream_t)stream, B, T, C, x, mix_x, x_mix));
}

int wkv6_shift_mix_five(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t R,
                        const void *x, const void *h, const void *w2t, const float *bias,
                        void *xr, void *xk, void *xv, void *xw, void *xg) {
    const int rc = check_mix(dtype, B, T, C, R);
    if (rc != WKV6_OK) return rc;
    if (!x || !h || !w2t || !bias || !xr || !xk || !xv || !xw || !xg) return WKV6_ERR_ARG;
    if (!aligned16(x) || !aligned16(h) || !aligned16(w2t) || !aligned16(bias) || !aligned16(xr) || !aligned16(xk) || !aligned16(xv) ||
        !aligned16(xw) || !aligned16(xg)) return WKV6_ERR_ARG;
    void *const out[5] = {xr, xk, xv, xw, xg};
    return finish(wkv6::shift_mix_five((hipStream_t)stream, B, T, C, R, x, h, w2t, bias, out));
}

int wkv6_shift_mix_five_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t R,
                                 const void *x, const void *h, const void *w2t, const float *bias,
                                 const void *gxr, const void *gxk, const void *gxv, const void *gxw, const void *gxg,
                                 void *gcoef, int64_t gcoef_stride, void *gp, void *gxx) {
    const int rc = check_mix(dtype, B, T, C, R);
    if (rc != WKV6_OK) return rc;
    if (!x || !h || !w2t || !bias || !gxr || !gxk || !gxv || !gxw || !gxg || !gcoef || !gp || !gxx) return WKV6_ERR_ARG;
    if (gcoef_stride < B * T * C || gcoef_stride % 8 != 0) return WKV6_ERR_ARG;
    if (!aligned16(x) || !aligned16(h) || !aligned16(w2t) || !aligned16(bias) || !aligned16(gxr) || !aligned16(gxk) || !aligned16(gxv) ||
        !aligned16(gxw) || !aligned16(gxg) || !aligned16(gcoef) || !aligned16(gp) || !aligned16(gxx)) return WKV6_ERR_ARG;
    const void *const gout[5] = {gxr, gxk, gxv, gxw, gxg};
    return finish(wkv6::shift_mix_five_backward((hipStream_t)stream, B, T, C, R, x, h, w2t, bias, gout, gcoef, gcoef_stride, gp, gxx));
}

int wkv6_shift_mix_x_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C,
                              const void *x, const float *mix_x, const void *gp, const void *gxx, const void *gxm,
                              void *gx, float *gmix_x) {
    const int rc = check_mix(dtype, B, T, C, 32);
    if (rc != WKV6_OK) return rc;
    if (!x || !mix_x || !gxm || !gx || !gmix_x || (gp == nullptr) != (gxx == nullptr)) return WKV6_ERR_ARG;
    if (!aligned16(x) || !aligned16(mix_x) || !aligned16(gp) || !aligned16(gxx) || !aligned16(gxm) || !aligned16(gx) || !aligned16(gmix_x))
        return WKV6_ERR_ARG;
    return finish(wkv6::shift_mix_x_backward((hipStream_t)stream, B, T, C, x, mix_x, gp, gxx, gxm, gx, gmix_x));
}

// Size of the part of the saved block that the kernels of one pass use (chunk states, arrival
// counters; sized so that the guarded per-timestep pass of the backward can use the same buffer).
static size_t saved_base_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    const size_t ws = wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H), sv = wkv6::chunk_saved_bytes(B, T, H);
    return ((ws > sv ? ws : sv) + 255) & ~(size_t)255;
}
// Segments the training pair of this shape runs in (1: one piece).  A (B,T,C) tensor cut into P
// segments is handled as a (B*P, T/P, C) tensor, so the base part is sized for that shape.
static int train_segments(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    const bool chunk = (algo == WKV6_ALGO_CHUNK && chunk_possible(dtype, T, C)) ||
                       (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    return chunk ? wkv6::chunk_train_segments(B, T, H) : 1;
}

// fp16 training pair: the bf16 copies of v and gy sit behind the base part of the saved block
static size_t f16_stage_offset(int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    const size_t ws = wkv6::scan_backward_workspace_bytes(B, T, C), cw = wkv6::chunk_backward_workspace_bytes(B, T, H),
                 sv = wkv6::chunk_saved_bytes(B, T, H);
    const size_t m = ws > cw ? (ws > sv ? ws : sv) : (cw > sv ? cw : sv);
    (void)algo;
    return (m + 255) & ~(size_t)255;
}

size_t wkv6_saved_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    if (check_shape(dtype, B, T, C, H) != WKV6_OK) return 0;
    if (train_chunk32(dtype, algo, B, T, H)) return wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H);
    if (dtype == WKV6_F16)
        return train_chunk(dtype, algo, T, C) ? f16_stage_offset(algo, B, T, C, H) + 2 * (size_t)(B * T * C) * 2 : 0;
    const bool chunk = (algo == WKV6_ALGO_CHUNK && chunk_possible(dtype, T, C)) ||
                       (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    if (!chunk) return 0;
    const int P = train_segments(dtype, algo, B, T, C, H);
    if (P > 1)
        return saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H) + wkv6::train_segments_layout(B, T, H, nullptr).bytes;
    const size_t ws = wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H), sv = wkv6::chunk_saved_bytes(B, T, H);
    return ws > sv ? ws : sv;
}

int wkv6_forward_save(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                      const void *r, const void *k, const void *v, const void *w, const void *u,
                      void *y, void *saved, size_t saved_bytes) {
    const size_t need = wkv6_saved_bytes(dtype, algo, B, T, C, H);
    if (need > 0 && (!saved || saved_bytes < need || !aligned16(saved))) return WKV6_ERR_WORKSPACE;
    if (need > 0 && dtype == WKV6_F16 && !train_chunk32(dtype, algo, B, T, H)) {
        if (algo < WKV6_ALGO_AUTO || algo > WKV6_ALGO_CHUNK) return WKV6_ERR_ARG;
        if (!r || !k || !v || !w || !u || !y) return WKV6_ERR_ARG;
        if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(y)) return WKV6_ERR_ARG;
        void *v_bf16 = reinterpret_cast<char *>(saved) + f16_stage_offset(algo, B, T, C, H);
        hipError_t e = wkv6::convert_to_bf16((hipStream_t)stream, wkv6::kF16, v, v_bf16, B * T * C);
        if (e != hipSuccess) return finish(e);
        return finish(wkv6::chunk_forward_save_f16((hipStream_t)stream, B, T, H, r, k, v, v_bf16, w, u, y, saved));
    }
    if (need > 0 && train_segments(dtype, algo, B, T, C, H) > 1) {
        // few pairs, long sequence: time segments side by side
        const int P = train_segments(dtype, algo, B, T, C, H);
        if (!r || !k || !v || !w || !u || !y) return WKV6_ERR_ARG;
        if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(y)) return WKV6_ERR_ARG;
        char *extra = reinterpret_cast<char *>(saved) + saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H);
        return finish(wkv6::chunk_forward_save_segments((hipStream_t)stream, B, T, H, r, k, v, w, u, y, saved, extra));
    }
    return forward_impl(stream, dtype, out_type(dtype), algo, B, T, C, H, 0, nullptr, r, k, v, w, u, nullptr, y, nullptr,
                        need > 0 ? saved : nullptr);
}

int wkv6_forward_with_state(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                            int has_init_state, const int64_t *state_map,
                            const void *r, const void *k, const void *v, const void *w, const void *u,
                            const void *s, void *y, void *ys) {
    if (!ys) return WKV6_ERR_ARG;
    return wkv6_forward_with_state_ex(stream, dtype, out_type(dtype), WKV6_ALGO_AUTO, B, T, C, H, has_init_state,
                                      state_map, r, k, v, w, u, s, y, ys, nullptr, 0);
}

int wkv6_forward_ex(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                    const void *r, const void *k, const void *v, const void *w, const void *u,
                    void *y, void *workspace, size_t workspace_bytes) {
    return wkv6_forward_with_state_ex(stream, dtype, out_type(dtype), algo, B, T, C, H, 0, nullptr,
                                      r, k, v, w, u, nullptr, y, nullptr, workspace, workspace_bytes);
}

int wkv6_forward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                 const void *r, const void *k, const void *v, const void *w, const void *u, void *y) {
    return wkv6_forward_ex(stream, dtype, WKV6_ALGO_AUTO, B, T, C, H, r, k, v, w, u, y, nullptr, 0);
}

// Workspace of a backward without saved states that runs in time segments (0: it does not): the
// saved-states block of the (B*P, T/P, C) shape, then the segments' states.
static size_t segments_workspace_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    const int P = train_segments(dtype, algo, B, T, C, H);
    if (P <= 1) return 0;
    return saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H) + wkv6::train_segments_layout(B, T, H, nullptr).bytes;
}

size_t wkv6_backward_workspace_bytes_ex(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    if (check_shape_any(dtype, B, T, C, H) == kSmallHead) return wkv6::generic_backward_workspace_bytes(B, T, C);
    if (check_shape(dtype, B, T, C, H) != WKV6_OK) return 0;
    // The per-timestep path keeps one fp32 per element (P), the chunked path one fp32 state per
    // 64-token chunk (which a workgroup's exact second pass reuses for its own P).
    size_t need = wkv6::scan_backward_workspace_bytes(B, T, C);
    if (train_chunk32(dtype, algo, B, T, H)) {   // one fp32 state per 32-token chunk
        const size_t c = wkv6::chunk32_saved_bytes(B, T, H);
        return c > need ? c : need;
    }
    if (algo == WKV6_ALGO_CHUNK || (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C))) {
        const size_t c = wkv6::chunk_backward_workspace_bytes(B, T, H);
        if (c > need) need = c;
        // few pairs, long sequence: the backward runs in time segments and keeps their states here
        const size_t seg = segments_workspace_bytes(dtype, algo, B, T, C, H);
        if (seg > need) need = seg;
    }
    return need;
}

size_t wkv6_backward_workspace_bytes(int dtype, int64_t B, int64_t T, int64_t C, int64_t H) {
    return wkv6_backward_workspace_bytes_ex(dtype, WKV6_ALGO_AUTO, B, T, C, H);
}

// backward_saved / backward_saved_sum of a shape whose training pair runs in time segments
static int backward_segments_impl(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                                  const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                                  void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum, void *saved, size_t saved_bytes) {
    if (!r || !k || !v || !w || !u || !gy || !gr || !gk || !gv || !gw || !gu) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gy) || !aligned16(gr) ||
        !aligned16(gk) || !aligned16(gv) || !aligned16(gw)) return WKV6_ERR_ARG;
    if (!saved || saved_bytes < wkv6_saved_bytes(dtype, algo, B, T, C, H) || !aligned16(saved)) return WKV6_ERR_WORKSPACE;
    const int P = train_segments(dtype, algo, B, T, C, H);
    char *extra = reinterpret_cast<char *>(saved) + saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H);
    return finish(wkv6::chunk_backward_saved_segments((hipStream_t)stream, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, gu_sum,
                                                      saved, extra));
}

static int backward_impl(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, size_t workspace_bytes,
                         bool states_ready, void *gu_sum = nullptr) {
    int rc = check_shape_any(dtype, B, T, C, H);
    if (rc != WKV6_OK && rc != kSmallHead) return rc;
    if (!r || !k || !v || !w || !u || !gy || !gr || !gk || !gv || !gw || !gu) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gy) || !aligned16(gr) ||
        !aligned16(gk) || !aligned16(gv) || !aligned16(gw)) return WKV6_ERR_ARG;
    if (algo < WKV6_ALGO_AUTO || algo > WKV6_ALGO_CHUNK) return WKV6_ERR_ARG;
    const size_t need = wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H);
    if (need > 0 && (!workspace || workspace_bytes < need || !aligned16(workspace))) return WKV6_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    if (rc == kSmallHead) {
        if (algo == WKV6_ALGO_CHUNK) return WKV6_ERR_UNSUPPORTED;
        rc = finish(wkv6::generic_backward(st, dtype, B, T, H, C / H, r, k, v, w, u, nullptr, gy, nullptr, gr, gk, gv, gw, gu, nullptr, workspace));
        if (rc == WKV6_OK && gu_sum) rc = finish(wkv6::sum_over_batch(st, out_type(dtype), B, C, gu, gu_sum));
        return rc;
    }
    if (train_chunk32(dtype, algo, B, T, H)) {
        // without saved states: a forward pass that only leaves the chunk states in the workspace
        if (!states_ready) {
            rc = finish(wkv6::chunk32_forward(st, dtype, WKV6_F32, B, T, H, r, k, v, w, u, nullptr, nullptr, nullptr, nullptr, workspace));
            if (rc != WKV6_OK) return rc;
        }
        rc = finish(wkv6::chunk32_backward(st, dtype, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace));
        if (rc == WKV6_OK && gu_sum) rc = finish(wkv6::sum_over_batch(st, out_type(dtype), B, C, gu, gu_sum));
        return rc;
    }
    if (algo == WKV6_ALGO_CHUNK && !chunk_possible(dtype, T, C)) return WKV6_ERR_UNSUPPORTED;
    const bool chunk = algo == WKV6_ALGO_CHUNK ||
                       (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    if (!chunk) {
        rc = finish(wkv6::scan_backward(st, dtype, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace));
        if (rc == WKV6_OK && gu_sum) rc = finish(wkv6::sum_over_batch(st, out_type(dtype), B, C, gu, gu_sum));
        return rc;
    }
    if (!states_ready && train_segments(dtype, algo, B, T, C, H) > 1) {
        const int P = train_segments(dtype, algo, B, T, C, H);
        char *extra = reinterpret_cast<char *>(workspace) + saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H);
        return finish(wkv6::chunk_backward_state_segments(st, B, T, H, r, k, v, w, u, nullptr, gy, nullptr, gr, gk, gv, gw, gu, nullptr,
                                                          workspace, extra));
    }
    return finish(wkv6::chunk_backward(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace, states_ready,
                                       states_ready ? gu_sum : nullptr));
}

int wkv6_backward_ex(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                     const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                     void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, size_t workspace_bytes) {
    return backward_impl(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace,
                         workspace_bytes, false);
}

// fp16 training pair, backward: gy (fp32) gets its bf16 copy next to the one of v the forward left
static int backward_saved_f16(void *stream, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                              const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                              void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum, void *saved, size_t saved_bytes) {
    if (!r || !k || !v || !w || !u || !gy || !gr || !gk || !gv || !gw || !gu) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gy) || !aligned16(gr) ||
        !aligned16(gk) || !aligned16(gv) || !aligned16(gw)) return WKV6_ERR_ARG;
    if (!saved || saved_bytes < wkv6_saved_bytes(WKV6_F16, algo, B, T, C, H) || !aligned16(saved)) return WKV6_ERR_WORKSPACE;
    char *v_bf16 = reinterpret_cast<char *>(saved) + f16_stage_offset(algo, B, T, C, H);
    char *gy_bf16 = v_bf16 + (size_t)(B * T * C) * 2;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = wkv6::convert_to_bf16(st, wkv6::kF32, gy, gy_bf16, B * T * C);
    if (e != hipSuccess) return finish(e);
    return finish(wkv6::chunk_backward(st, B, T, H, r, k, v_bf16, w, u, gy_bf16, gr, gk, gv, gw, gu, saved, true, gu_sum,
                                       nullptr, nullptr, nullptr, wkv6::kF16, v, gy));
}

int wkv6_backward_saved(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                        const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                        void *gr, void *gk, void *gv, void *gw, void *gu, void *saved, size_t saved_bytes) {
    // `saved` doubles as the workspace: the guarded per-timestep pass only runs when the chunked
    // results (and with them the saved states) are discarded anyway
    if (check_shape(dtype, B, T, C, H) == WKV6_OK && algo >= WKV6_ALGO_AUTO && algo <= WKV6_ALGO_CHUNK &&
        dtype == WKV6_F16 && train_chunk(dtype, algo, T, C))
        return backward_saved_f16(stream, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, nullptr, saved, saved_bytes);
    if (check_shape(dtype, B, T, C, H) == WKV6_OK && algo >= WKV6_ALGO_AUTO && algo <= WKV6_ALGO_CHUNK &&
        train_segments(dtype, algo, B, T, C, H) > 1)
        return backward_segments_impl(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, nullptr, saved, saved_bytes);
    return backward_impl(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, saved, saved_bytes,
                         wkv6_saved_bytes(dtype, algo, B, T, C, H) > 0);
}

int wkv6_backward_saved_sum(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                            const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                            void *gr, void *gk, void *gv, void *gw, void *gu, void *gu_sum,
                            void *saved, size_t saved_bytes) {
    if (!gu_sum) return WKV6_ERR_ARG;
    if (check_shape(dtype, B, T, C, H) == WKV6_OK && algo >= WKV6_ALGO_AUTO && algo <= WKV6_ALGO_CHUNK &&
        dtype == WKV6_F16 && train_chunk(dtype, algo, T, C))
        return backward_saved_f16(stream, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, gu_sum, saved, saved_bytes);
    if (check_shape(dtype, B, T, C, H) == WKV6_OK && algo >= WKV6_ALGO_AUTO && algo <= WKV6_ALGO_CHUNK &&
        train_segments(dtype, algo, B, T, C, H) > 1)
        return backward_segments_impl(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, gu_sum, saved, saved_bytes);
    const size_t need = wkv6_saved_bytes(dtype, algo, B, T, C, H);
    if (need > 0 && saved_bytes < need) return WKV6_ERR_WORKSPACE;
    return backward_impl(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, saved, saved_bytes,
                         need > 0, gu_sum);
}

// where the pairs' final states sit in the workspace of a full-precision backward with state gradients
static size_t state32_offset(int64_t B, int64_t T, int64_t H) { return (wkv6::chunk32_saved_bytes(B, T, H) + 255) & ~(size_t)255; }

size_t wkv6_backward_with_state_workspace_bytes(int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H) {
    if (check_shape_any(dtype, B, T, C, H) == kSmallHead) return wkv6::generic_backward_workspace_bytes(B, T, C);
    if (check_shape(dtype, B, T, C, H) != WKV6_OK) return 0;
    size_t need = wkv6::scan_backward_state_workspace_bytes(B, T, C);
    const size_t c = wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H);
    if (c > need) need = c;
    if (train_chunk32(dtype, algo, B, T, H)) {   // the chunk states, then the final state of every pair
        const size_t s = state32_offset(B, T, H) + (size_t)(B * H) * 64 * 64 * sizeof(float);
        if (s > need) need = s;
    }
    return need;   // (includes the segments' states where the backward runs in time segments)
}

int wkv6_backward_with_state(void *stream, int dtype, int algo, int64_t B, int64_t T, int64_t C, int64_t H,
                             const void *r, const void *k, const void *v, const void *w, const void *u,
                             const float *s0, const void *gy, const float *gsT,
                             void *gr, void *gk, void *gv, void *gw, void *gu, float *gs0,
                             void *workspace, size_t workspace_bytes) {
    int rc = check_shape_any(dtype, B, T, C, H);
    if (rc != WKV6_OK && rc != kSmallHead) return rc;
    if (!r || !k || !v || !w || !u || !gy || !gr || !gk || !gv || !gw || !gu) return WKV6_ERR_ARG;
    if (!aligned16(r) || !aligned16(k) || !aligned16(v) || !aligned16(w) || !aligned16(gy) || !aligned16(gr) ||
        !aligned16(gk) || !aligned16(gv) || !aligned16(gw)) return WKV6_ERR_ARG;
    if ((s0 && !aligned16(s0)) || (gsT && !aligned16(gsT)) || (gs0 && !aligned16(gs0))) return WKV6_ERR_ARG;
    if (algo < WKV6_ALGO_AUTO || algo > WKV6_ALGO_CHUNK) return WKV6_ERR_ARG;
    const size_t need = wkv6_backward_with_state_workspace_bytes(dtype, algo, B, T, C, H);
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) return WKV6_ERR_WORKSPACE;
    if (rc == kSmallHead) {
        if (algo == WKV6_ALGO_CHUNK) return WKV6_ERR_UNSUPPORTED;
        return finish(wkv6::generic_backward((hipStream_t)stream, dtype, B, T, H, C / H, r, k, v, w, u, s0, gy, gsT, gr, gk, gv, gw, gu, gs0, workspace));
    }
    if (algo == WKV6_ALGO_CHUNK && !chunk_possible(dtype, T, C)) return WKV6_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (train_chunk32(dtype, algo, B, T, H)) {
        // full-precision chunk form: the chunk states (and the final one, which anchors the decay gradient's sums
        // where a gradient arrives at it) from a states-only forward that starts from s0, then the backward
        float *sT = gsT ? reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + state32_offset(B, T, H)) : nullptr;
        const hipError_t e = wkv6::chunk32_forward(st, dtype, WKV6_F32, B, T, H, r, k, v, w, u, s0, nullptr, nullptr, sT, workspace);
        if (e != hipSuccess) return finish(e);
        return finish(wkv6::chunk32_backward(st, dtype, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace, s0, gsT, sT, gs0));
    }
    const bool chunk = algo == WKV6_ALGO_CHUNK || (algo == WKV6_ALGO_AUTO && chunk_eligible(dtype, T, C));
    if (!chunk)
        return finish(wkv6::scan_backward_state(st, dtype, B, T, H, r, k, v, w, u, s0, gy, gsT, gr, gk, gv, gw, gu, gs0, workspace));
    const int P = train_segments(dtype, algo, B, T, C, H);
    if (P > 1) {
        char *extra = reinterpret_cast<char *>(workspace) + saved_base_bytes(dtype, WKV6_ALGO_CHUNK, B * P, T / P, C, H);
        return finish(wkv6::chunk_backward_state_segments(st, B, T, H, r, k, v, w, u, s0, gy, gsT, gr, gk, gv, gw, gu, gs0,
                                                          workspace, extra));
    }
    return finish(wkv6::chunk_backward(st, B, T, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace, false, nullptr,
                                       s0, gsT, gs0));
}

int wkv6_backward(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                  const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                  void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, size_t workspace_bytes) {
    return wkv6_backward_ex(stream, dtype, WKV6_ALGO_AUTO, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu,
                            workspace, workspace_bytes);
}

int wkv6_backward_static(void *stream, int dtype, int64_t B, int64_t T, int64_t C, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu) {
    const int rc = check_shape(dtype, B, T, C, H);
    if (rc != WKV6_OK) return rc;
    int algo = WKV6_ALGO_AUTO;
    size_t need = wkv6_backward_workspace_bytes(dtype, B, T, C, H);
    if (need > WKV6_STATIC_SCRATCH_BYTES) {   // the per-timestep kernels keep less
        algo = WKV6_ALGO_SCAN;
        need = wkv6_backward_workspace_bytes_ex(dtype, algo, B, T, C, H);
    }
    if (need > WKV6_STATIC_SCRATCH_BYTES) return WKV6_ERR_WORKSPACE;   // larger than the library's own array
    hipError_t e = hipSuccess;
    void *ws = static_scratch(&e);
    if (ws == nullptr) return finish(e);
    // (the workspace needs no initial contents; what the last call left in it is overwritten)
    return wkv6_backward_ex(stream, dtype, algo, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, ws, WKV6_STATIC_SCRATCH_BYTES);
}

// ---- XLA custom-call surface ------------------------------------------------------------

size_t wkv6_create_descriptor(int B, int T, int C, int H, int S, int x_type, int y_type, void *out) {
    static_assert(sizeof(wkv6_descriptor) == 28, "descriptor must stay 28 bytes");
    wkv6_descriptor d;
    memset(&d, 0, sizeof d);
    d.B = B; d.T = T; d.C = C; d.H = H; d.S = S ? 1 : 0; d.x_type = x_type; d.y_type = y_type;
    if (out) memcpy(out, &d, sizeof d);
    return sizeof d;
}

static bool unpack(const char *opaque, size_t len, wkv6_descriptor *d) {
    if (!opaque || len != sizeof(wkv6_descriptor)) { g_last_status = WKV6_ERR_ARG; return false; }
    memcpy(d, opaque, sizeof *d);
    if (d->y_type != out_type(d->x_type)) { g_last_status = WKV6_ERR_ARG; return false; }
    return true;
}

void wkv_forward(void *stream, void **buffers, const char *opaque, size_t opaque_len) {
    wkv6_descriptor d;
    if (!unpack(opaque, opaque_len, &d) || !buffers) { g_last_status = WKV6_ERR_ARG; return; }
    g_last_status = wkv6_forward(stream, d.x_type, d.B, d.T, d.C, d.H, buffers[0], buffers[1], buffers[2],
                                 buffers[3], buffers[4], buffers[5]);
}

void wkv_backward(void *stream, void **buffers, const char *opaque, size_t opaque_len) {
    wkv6_descriptor d;
    if (!unpack(opaque, opaque_len, &d) || !buffers) { g_last_status = WKV6_ERR_ARG; return; }
    g_last_status = wkv6_backward(stream, d.x_type, d.B, d.T, d.C, d.H, buffers[0], buffers[1], buffers[2],
                                  buffers[3], buffers[4], buffers[5], buffers[6], buffers[7], buffers[8],
                                  buffers[9], buffers[10], buffers[11],
                                  wkv6_backward_workspace_bytes(d.x_type, d.B, d.T, d.C, d.H));
}

void wkv_forward_with_state(void *stream, void **buffers, const char *opaque, size_t opaque_len) {
    wkv6_descriptor d;
    if (!unpack(opaque, opaque_len, &d) || !buffers) { g_last_status = WKV6_ERR_ARG; return; }
    if (d.S) {
        g_last_status = wkv6_forward_with_state(stream, d.x_type, d.B, d.T, d.C, d.H, 1,
                                                (const int64_t *)buffers[0], buffers[1], buffers[2], buffers[3],
                                                buffers[4], buffers[5], buffers[6], buffers[7], buffers[8]);
    } else {
        g_last_status = wkv6_forward_with_state(stream, d.x_type, d.B, d.T, d.C, d.H, 0, nullptr, buffers[0],
                                                buffers[1], buffers[2], buffers[3], buffers[4], nullptr,
                                                buffers[5], buffers[6]);
    }
}

void wkv_forward_save(void *stream, void **buffers, const char *opaque, size_t opaque_len) {
    wkv6_descriptor d;
    if (!unpack(opaque, opaque_len, &d) || !buffers) { g_last_status = WKV6_ERR_ARG; return; }
    const size_t n = wkv6_saved_bytes(d.x_type, WKV6_ALGO_AUTO, d.B, d.T, d.C, d.H);
    if (n == 0) { g_last_status = WKV6_ERR_UNSUPPORTED; return; }   // (nothing to save: the caller uses wkv_forward)
    g_last_status = wkv6_forward_save(stream, d.x_type, WKV6_ALGO_AUTO, d.B, d.T, d.C, d.H, buffers[0], buffers[1], buffers[2],
                                      buffers[3], buffers[4], buffers[5], buffers[6], n);
}

void wkv_backward_saved(void *stream, void **buffers, const char *opaque, size_t opaque_len) {
    wkv6_descriptor d;
    if (!unpack(opaque, opaque_len, &d) || !buffers) { g_last_status = WKV6_ERR_ARG; return; }
    const size_t n = wkv6_saved_bytes(d.x_type, WKV6_ALGO_AUTO, d.B, d.T, d.C, d.H);
    if (n == 0) { g_last_status = WKV6_ERR_UNSUPPORTED; return; }
    // the block the call works on is the result that the caller aliases to the operand `saved`; if the two
    // are different buffers after all, the operand stays as it is and the result starts as its copy
    if (buffers[12] != buffers[6]) {
        const hipError_t e = hipMemcpyAsync(buffers[12], buffers[6], n, hipMemcpyDeviceToDevice, (hipStream_t)stream);
        if (e != hipSuccess) { g_last_status = finish(e); return; }
    }
    g_last_status = wkv6_backward_saved_sum(stream, d.x_type, WKV6_ALGO_AUTO, d.B, d.T, d.C, d.H, buffers[0], buffers[1], buffers[2],
                                            buffers[3], buffers[4], buffers[5], buffers[7], buffers[8], buffers[9],
                                            buffers[10], buffers[11], buffers[13], buffers[12], n);
}

}  // extern "C"
