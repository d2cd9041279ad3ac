// Host-side launchers of the WKV6 kernels (internal to the library; the public ABI is include/wkv6.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace wkv6 {

enum { kBF16 = 0, kF16 = 1, kF32 = 2 };  // same numbering as the public header

// A kernel launched "behind a gate" does nothing unless *flag == epoch.  The chunked kernels raise
// the flag (write `epoch`) when a tile's decay leaves the range their scaling can represent; the
// exact per-timestep kernels enqueued after them on the same stream then redo the whole call.
// Epochs are unique per call, so the flag word never needs clearing.
struct Gate {
    const unsigned long long *flag;   // nullptr: always open
    unsigned long long epoch;
    __device__ __forceinline__ bool closed() const { return flag != nullptr && *flag != epoch; }
};

// --- per-timestep recurrence (wkv6_scan.hip) ---
hipError_t scan_forward(hipStream_t st, int dtype, int state_dtype, int64_t B, int64_t T, int64_t H,
                        const void *r, const void *k, const void *v, const void *w, const void *u,
                        const void *s0, const int64_t *map, void *y, void *sT, Gate gate);
size_t scan_backward_workspace_bytes(int64_t B, int64_t T, int64_t C);
hipError_t scan_backward(hipStream_t st, int dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                         void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, Gate gate);

// --- chunk-parallel MFMA form, bf16 tensors only (wkv6_chunk.hip) ---
hipError_t chunk_forward(hipStream_t st, int state_dtype, int64_t B, int64_t T, int64_t H,
                         const void *r, const void *k, const void *v, const void *w, const void *u,
                         const void *s0, const int64_t *map, void *y, void *sT, void *saved_states,
                         unsigned long long *wild_flag, unsigned long long epoch);

size_t chunk_backward_workspace_bytes(int64_t B, int64_t T, int64_t H);
// states_ready: the workspace already holds the chunk-start states (written by a forward pass)
hipError_t chunk_backward(hipStream_t st, int64_t B, int64_t T, int64_t H,
                          const void *r, const void *k, const void *v, const void *w, const void *u, const void *gy,
                          void *gr, void *gk, void *gv, void *gw, void *gu, void *workspace, bool states_ready,
                          unsigned long long *wild_flag, unsigned long long epoch);

}  // namespace wkv6
