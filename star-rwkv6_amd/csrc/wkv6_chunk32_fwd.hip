// Forward of the full-precision chunk form (see wkv6_chunk32.h for the algebra): fp32 and fp16 tensors,
// every product on v_mfma_f32_16x16x4_f32, relative error that of fp32.
//
// One workgroup of twelve waves per (batch, head) pair.  Waves 4..11 load, in two groups of four that take
// the chunks in turn: a group brings its chunk from global memory (16-byte loads issued two chunks ahead,
// converted to fp32), forms the decay products with row-wide DPP steps and writes the operand tiles to LDS.
// Waves 0..3 compute: wave q owns value columns 16q..16q+15 of the state (four 16x16 accumulator tiles
// over the key rows), which never leaves its registers: as a C/D tile it is directly the B operand of
// R' S.  Two workgroup barriers per chunk:
//   phase 1  compute: y = R' S ; three of the waves form one tile each of A = R~ K~^T (masked, with the
//            u diagonal) -> LDS ; y rows of the chunk behind LDS -> global      load: tiles R', K', V, e^{c_32} of the next chunk -> LDS
//   phase 2  compute: y += A V -> LDS ;  S = e^{c_32} o S + K'^T V     load: tiles R~, K~ of the next chunk -> LDS;
//            the operands of the chunk after it formed in registers (decay products over the rows)
// Saved states (one per chunk, for the backward) are written in fragment order: tile (q, ib) as 64 lanes
// x 4 consecutive floats, element v of lane (n, g) = S[16 ib + 4g + v][16q + n].
#include "wkv6_chunk32.h"
#include "wkv6_kernels.h"
#include "wkv6_scan_body.h"

#include <type_traits>

// groups of loading waves that take the chunks in turn (three measured no faster than two)
constexpr int kC32FwdGroups = 2;

namespace wkv6 {

// The value is final here: what computes it stays in front of this point and what reads it behind it.
__device__ __forceinline__ void pin_value(float &x) { asm volatile("" : "+v"(x)); }

struct C32FwdLds {
    float Rp[2][kC32][kLd], Kp[2][kC32][kLd], V[2][kC32][kLd];   // R', K', v of the chunk in hand and the next
    float Rm[kC32][kLd], Km[kC32][kLd];                          // R~, K~
    float Y[kC32][kLd];                                          // finished y rows on their way out
    float A[kC32][kLa];
    float e_all[2][kN];                                          // e^{c_32}
    float ruk[4][kC32];                                          // sum_i r u k over each loading wave's channels
    int wild[4 * 3];
};
union C32FwdSmem {
    C32FwdLds chunk;
    ScanFwdLdsT<8> scan;
};

struct C32FwdArgs {
    int T, H;
    const void *r, *k, *v, *w, *u, *s0;
    const int64_t *map;
    void *y, *sT;
    float *saved;   // [pair][chunk][4096] chunk-start states in fragment order (null: not kept)
};

// kOut = false: only the states (chunk states and / or the final one): no y, no R-side operands
template <typename Tin, typename Tout, typename Ts, int kGroups, bool kOut>
__global__ __launch_bounds__(256 + 256 * kGroups) void chunk32_fwd_kernel(const C32FwdArgs a)
{
    extern __shared__ __align__(16) unsigned char c32_smem[];
    C32FwdLds &L = reinterpret_cast<C32FwdSmem *>(c32_smem)->chunk;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int T = a.T, H = a.H;
    const int pair = blockIdx.x, b = pair / H, h = pair - b * H;
    const int64_t C = (int64_t)H * kN;
    const int64_t base = (int64_t)b * T * C + (int64_t)h * kN;
    const int nchunk = (T + kC32 - 1) / kC32;
    const Tin *r = reinterpret_cast<const Tin *>(a.r), *k = reinterpret_cast<const Tin *>(a.k);
    const Tin *v = reinterpret_cast<const Tin *>(a.v), *w = reinterpret_cast<const Tin *>(a.w);
    const Tin *u = reinterpret_cast<const Tin *>(a.u);
    Tout *y = reinterpret_cast<Tout *>(a.y);

    if (wave >= 4) {
        // ---------------- loading waves ----------------
        const int grp = (wave - 4) >> 2, p = (wave - 4) & 3, t16 = lane & 15, ch = 16 * p + 4 * (lane >> 4);
        float fu[4];
        load4(u + h * kN + ch, fu);
        Raw4<Tin> nr[2], nk[2], nv[2], nw[2];   // the group's next chunk on its way in, as loaded
        auto fetch = [&](int c) {
            const int64_t row0 = base + (int64_t)c * kC32 * C;   // (uniform)
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int o = min(16 * x + t16, T - 1 - c * kC32) * (int)C + ch;   // rows past the end read the last one
                nr[x].load(r + row0 + o); nk[x].load(k + row0 + o); nv[x].load(v + row0 + o); nw[x].load(w + row0 + o);
            }
        };
        // the chunk whose operands are formed: two channels of the lane's four at a time (a barrier in between)
        float op_r[2][4], op_k[2][4], op_v[2][4], hm_r[2][4], hm_k[2][4], e_all[4], part[2];
        bool wild = false;
        auto form = [&](auto half, int c) {
            constexpr int E0 = 2 * decltype(half)::value;
            const bool valid[2] = {c * kC32 + t16 < T, c * kC32 + 16 + t16 < T};
            C32Scale sc;
            sc.wild = false;
            float d[2][4], fw[2][4];
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int e = E0; e < E0 + 2; ++e) fw[x][e] = nw[x].at(e);
            c32_scale<E0, E0 + 2>(fw, valid, sc, d);
            wild |= sc.wild;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                float s = E0 == 0 ? 0.f : part[x];
#pragma unroll
                for (int e = E0; e < E0 + 2; ++e) {
                    const float fr = valid[x] ? nr[x].at(e) : 0.f, fk = valid[x] ? nk[x].at(e) : 0.f;
                    op_k[x][e] = fk * sc.kp[x][e];
                    if (kOut) {
                        op_r[x][e] = fr * sc.rp[x][e];
                        hm_r[x][e] = fr * sc.rm[x][e];
                        hm_k[x][e] = fk * sc.km[x][e];
                    }
                    op_v[x][e] = valid[x] ? nv[x].at(e) : 0.f;
                    e_all[e] = sc.all[e];
                    s = fmaf(fr * fk, fu[e], s);
                }
                if (kOut) part[x] = E0 == 0 ? s : sum_rows4(s);
            }
        };
        auto settle = [&](auto half) {
            constexpr int E0 = 2 * decltype(half)::value;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
#pragma unroll
                for (int e = E0; e < E0 + 2; ++e) {
                    pin_value(op_k[x][e]);
                    pin_value(op_v[x][e]);
                    if (kOut) { pin_value(op_r[x][e]); pin_value(hm_r[x][e]); pin_value(hm_k[x][e]); }
                }
                if (kOut) pin_value(part[x]);
            }
#pragma unroll
            for (int e = E0; e < E0 + 2; ++e) pin_value(e_all[e]);
        };
        const std::integral_constant<int, 0> h0;
        const std::integral_constant<int, 1> h1;
        auto publish = [&](int c) {
            const int buf = c & 1;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int t = 16 * x + t16;
                if (kOut) *reinterpret_cast<f32x4 *>(&L.Rp[buf][t][ch]) = (f32x4){op_r[x][0], op_r[x][1], op_r[x][2], op_r[x][3]};
                *reinterpret_cast<f32x4 *>(&L.Kp[buf][t][ch]) = (f32x4){op_k[x][0], op_k[x][1], op_k[x][2], op_k[x][3]};
                *reinterpret_cast<f32x4 *>(&L.V[buf][t][ch]) = (f32x4){op_v[x][0], op_v[x][1], op_v[x][2], op_v[x][3]};
            }
            if (t16 == 0) *reinterpret_cast<f32x4 *>(&L.e_all[buf][ch]) = (f32x4){e_all[0], e_all[1], e_all[2], e_all[3]};
        };
        auto finish = [&]() {
            if (!kOut) return;
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int t = 16 * x + t16;
                *reinterpret_cast<f32x4 *>(&L.Rm[t][ch]) = (f32x4){hm_r[x][0], hm_r[x][1], hm_r[x][2], hm_r[x][3]};
                *reinterpret_cast<f32x4 *>(&L.Km[t][ch]) = (f32x4){hm_k[x][0], hm_k[x][1], hm_k[x][2], hm_k[x][3]};
                if (lane < 16) L.ruk[p][t] = part[x];
            }
        };
        // Group j % kGroups brings chunk j: it forms the chunk's operands while chunk j - 2 is computed (its
        // loads are the only ones the wave has in flight, so the wait for them is exact), sends for its
        // next chunk, and hands the operands to LDS while chunk j - 1 is computed.
        if (grp < 2) {
            fetch(grp);
            form(h0, grp);
            form(h1, grp);
            if (grp == 0) { publish(0); finish(); }
            if (grp + kGroups < nchunk) fetch(grp + kGroups);
        } else if (grp < nchunk) fetch(grp);
        __syncthreads();
        for (int c = 0; c < nchunk; ++c) {
            const bool forming = (c + 2) % kGroups == grp && c + 2 < nchunk;
            const bool handing = (c + 1) % kGroups == grp && c + 1 < nchunk;
            if (forming) form(h0, c + 2);
            if (handing) publish(c + 1);
            __syncthreads();
            if (forming) {
                form(h1, c + 2);
                // (every value of this chunk is final before the next loads are issued: left to itself the compiler
                // moves the last products behind the loads, whose destinations are then other registers than the
                // ones still being read, and the copy back at the end of the iteration waits for the loads)
                settle(h1);
                if (c + 2 + kGroups < nchunk) fetch(c + 2 + kGroups);
            }
            if (handing) finish();
            __syncthreads();
        }
        const bool any = __any(wild);
        if (lane == 0) L.wild[wave - 4] = any;
    } else {
        // ---------------- computing waves ----------------
        const int q = wave, n = lane & 15, g = lane >> 4;
        typedef Ts StateT;
        f32x4 S[4];
        if (a.s0) {
            const int64_t row = a.map ? a.map[b] : (int64_t)b;
            const StateT *p0 = reinterpret_cast<const StateT *>(a.s0) + (row * H + h) * (kN * kN) + 16 * q + n;
#pragma unroll
            for (int ib = 0; ib < 4; ++ib)
#pragma unroll
                for (int e = 0; e < 4; ++e) S[ib][e] = load1(p0 + (16 * ib + 4 * g + e) * kN);
        } else {
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) S[ib] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
        // the y rows of a finished chunk, LDS -> global as whole 16-byte pieces (the loading waves keep to loads:
        // loads and stores of one wave complete in no fixed order, and a store in flight would make every
        // wait for a load a wait for everything)
        const int t16 = lane & 15, ch = 16 * q + 4 * (lane >> 4);
        auto store_y = [&](int c) {
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int t = c * kC32 + 16 * x + t16;
                const f32x4 o = *reinterpret_cast<const f32x4 *>(&L.Y[16 * x + t16][ch]);
                if (t < T) store4(y + base + (int64_t)t * C + ch, o[0], o[1], o[2], o[3]);
            }
        };
        float *saved = a.saved ? a.saved + (int64_t)pair * nchunk * (kN * kN) + (q * 4) * 256 + lane * 4 : nullptr;
        __syncthreads();
        for (int c = 0; c < nchunk; ++c) {
            const int buf = c & 1;
            if (kOut && c > 0 && y) store_y(c - 1);
            if (saved) {
#pragma unroll
                for (int ib = 0; ib < 4; ++ib) *reinterpret_cast<f32x4 *>(saved + (int64_t)c * (kN * kN) + ib * 256) = S[ib];
            }
            // phase 1: y = R' S, one tile of A
            f32x4 yt[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int tb = 0; kOut && tb < 2; ++tb)
#pragma unroll
                for (int ib = 0; ib < 4; ++ib) {
                    const f32x4 fr = *reinterpret_cast<const f32x4 *>(&L.Rp[buf][16 * tb + n][16 * ib + 4 * g]);
                    yt[tb] = mfma16(fr, S[ib], yt[tb]);
                }
            if (kOut && q < 3) {
                // tile (tb, sb) of A, computed transposed: lane (n, g) ends with A[16 tb + n][16 sb + 4g + v]
                const int tb = q == 0 ? 0 : 1, sb = q == 1 ? 1 : 0;
                f32x4 at = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ib = 0; ib < 4; ++ib) {
                    const f32x4 fk = *reinterpret_cast<const f32x4 *>(&L.Km[16 * sb + n][16 * ib + 4 * g]);
                    const f32x4 fr = *reinterpret_cast<const f32x4 *>(&L.Rm[16 * tb + n][16 * ib + 4 * g]);
                    at = mfma16(fk, fr, at);
                }
                if (tb == sb) {
                    const int t = 16 * tb + n;
                    const float diag = (L.ruk[0][t] + L.ruk[1][t]) + (L.ruk[2][t] + L.ruk[3][t]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) at[e] = (4 * g + e < n) ? at[e] : (4 * g + e == n ? diag : 0.f);
                }
                *reinterpret_cast<f32x4 *>(&L.A[16 * tb + n][16 * sb + 4 * g]) = at;
            }
            __syncthreads();
            // phase 2: y += A V ; S = e^{c_32} o S + K'^T V
            f32x4 fv[2];
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int e = 0; e < 4; ++e) fv[sb][e] = L.V[buf][16 * sb + 4 * g + e][16 * q + n];
#pragma unroll
            for (int tb = 0; kOut && tb < 2; ++tb)
#pragma unroll
                for (int sb = 0; sb <= tb; ++sb) {
                    const f32x4 fa = *reinterpret_cast<const f32x4 *>(&L.A[16 * tb + n][16 * sb + 4 * g]);
                    yt[tb] = mfma16(fa, fv[sb], yt[tb]);
                }
#pragma unroll
            for (int tb = 0; kOut && tb < 2; ++tb)
#pragma unroll
                for (int e = 0; e < 4; ++e) L.Y[16 * tb + 4 * g + e][16 * q + n] = yt[tb][e];
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) {
                const f32x4 ea = *reinterpret_cast<const f32x4 *>(&L.e_all[buf][16 * ib + 4 * g]);
                S[ib] *= ea;
#pragma unroll
                for (int sb = 0; sb < 2; ++sb) {
                    f32x4 fk;
#pragma unroll
                    for (int e = 0; e < 4; ++e) fk[e] = L.Kp[buf][16 * sb + 4 * g + e][16 * ib + n];
                    S[ib] = mfma16(fk, fv[sb], S[ib]);
                }
            }
            __syncthreads();
        }
        if (kOut && y) store_y(nchunk - 1);
        if (a.sT) {
            StateT *p0 = reinterpret_cast<StateT *>(a.sT) + (int64_t)pair * (kN * kN) + 16 * q + n;
#pragma unroll
            for (int ib = 0; ib < 4; ++ib)
#pragma unroll
                for (int e = 0; e < 4; ++e) store1(p0 + (16 * ib + 4 * g + e) * kN, S[ib][e]);
        }
    }
    __syncthreads();
    // a pair whose decay left the reach: once more, one timestep at a time
    int wild_any = 0;
#pragma unroll
    for (int i = 0; i < 4 * kGroups; ++i) wild_any |= L.wild[i];
    if (wild_any && (kOut || a.sT)) {   // (its chunk states are not used: the backward takes the same way out)
        __syncthreads();
        scan_fwd_body<Tin, Tout, Ts, 8>(reinterpret_cast<C32FwdSmem *>(c32_smem)->scan, b, h, T, H, r, k, v, w, u,
                                        reinterpret_cast<const Ts *>(a.s0), a.map, y, reinterpret_cast<Ts *>(a.sT));
    }
}

bool chunk32_forward_applies(int dtype, int64_t B, int64_t T, int64_t H) {
    return (dtype == kF32 || dtype == kF16) && T >= 2 * kC32 && B * H < ((int64_t)1 << 31) && T * H * kN < ((int64_t)1 << 31);
}
size_t chunk32_saved_bytes(int64_t B, int64_t T, int64_t H) {
    return (size_t)(B * H) * (size_t)((T + kC32 - 1) / kC32) * (kN * kN) * sizeof(float);
}

template <typename Tin, typename Tout, typename Ts, bool kOut>
static hipError_t launch(hipStream_t st, int64_t B, const C32FwdArgs &a) {
    constexpr int lds = (int)sizeof(C32FwdSmem);
    constexpr int kGroups = kC32FwdGroups;
    const hipError_t e = allow_dynamic_lds<chunk32_fwd_kernel<Tin, Tout, Ts, kGroups, kOut>>(lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((chunk32_fwd_kernel<Tin, Tout, Ts, kGroups, kOut>), dim3((unsigned)(B * a.H)), dim3(256 + 256 * kGroups), lds, st, a);
    return hipGetLastError();
}

hipError_t chunk32_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H,
                           const void *r, const void *k, const void *v, const void *w, const void *u,
                           const void *s0, const int64_t *map, void *y, void *sT, void *saved_states)
{
    (void)state_dtype;   // fp32 and fp16 tensors keep fp32 states
    C32FwdArgs a;
    a.T = (int)T; a.H = (int)H;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.map = map; a.y = y; a.sT = sT;
    a.saved = reinterpret_cast<float *>(saved_states);
    if (y == nullptr)
        return dtype == kF32 ? launch<float, float, float, false>(st, B, a) : launch<f16_t, float, float, false>(st, B, a);
    return dtype == kF32 ? launch<float, float, float, true>(st, B, a) : launch<f16_t, float, float, true>(st, B, a);
}

}  // namespace wkv6
