"""jax flavour of the WKV6 operator: jax.custom_vjp over the XLA custom-call targets of
libwkv6_gfx950.so.

Mirrors rwkv_kernel/jax_rwkv_kernel.py of the reference: same constructor and call signature,
residuals = the inputs (rwkv_fwd :68-71), gu summed over the batch (:166), output dtype rule
(:90-93), `seq_len <= max_sequence_length` assertion (:128).  The binding differs: instead of a
pybind module holding PyCapsules and jax.core.Primitive + jaxlib.hlo_helpers.custom_call (all
removed from current jax), the library's three status-less custom-call symbols
(wkv_forward / wkv_backward / wkv_forward_with_state, include/wkv6.h) are wrapped with
jax.ffi.pycapsule, registered for platform "ROCM" with api_version=0, and invoked through
jax.ffi.ffi_call(custom_call_api_version=2, legacy_backend_config=<28-byte descriptor>) --
the same opaque descriptor and buffer orders as the reference's lowering (:75-111, :172-218,
:358-376).  The backward call declares one extra result that XLA allocates as scratch.

Where the library has something worth keeping for the backward (the chunked kernels' per-chunk
states), the custom_vjp's forward rule runs the target wkv_forward_save, whose second result -- a
block of bytes -- joins the residuals, and the backward rule runs wkv_backward_saved, which skips the
forward state sweep and returns gu already summed over the batch.  The primal call outside of
differentiation stays wkv_forward.

jax is not installed in the image this library is developed in, so this module is exercised only
where jax (ROCm build) exists; importing it without jax raises ImportError.
"""
import ctypes
from functools import reduce

import jax
import jax.numpy as jnp
import numpy as np

from . import _native

_REGISTERED = False
_TARGETS = ("wkv_forward", "wkv_backward", "wkv_forward_with_state", "wkv_forward_save", "wkv_backward_saved")


def _register():
    global _REGISTERED
    if _REGISTERED:
        return
    lib = _native.load()
    for name in _TARGETS:
        fn = getattr(lib, name)
        jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(fn), platform="ROCM", api_version=0)
    _REGISTERED = True


def _code(dtype):
    dtype = jnp.dtype(dtype)
    if dtype == jnp.bfloat16:
        return _native.BF16
    if dtype == jnp.float16:
        return _native.F16
    if dtype == jnp.float32:
        return _native.F32
    raise AssertionError("r, k, v, w, u must be float32, float16 or bfloat16")


def _out_dtype(dtype):
    return jnp.float32 if jnp.dtype(dtype) == jnp.float16 else jnp.dtype(dtype)


class RWKVKernelOperator:
    def __init__(self, head_size, max_sequence_length):
        assert isinstance(head_size, int) and isinstance(max_sequence_length, int)
        assert head_size > 0 and max_sequence_length > 0
        assert head_size % 4 == 0, "head_size must be a multiple of 4"
        lib = _native.load()
        if not lib.wkv6_supports_head_size(head_size):
            raise _native.WKV6Error("libwkv6_gfx950 is built for head sizes 64 (all paths) and the other multiples of 4 up to 128 (plain calls), got %d" % head_size)
        _register()
        self.head_size = head_size
        self.max_sequence_length = max_sequence_length
        N = head_size

        def check(r, k, v, w, u):
            assert r.ndim == 3 and all(r.shape == x.shape for x in (k, v, w))
            B, T, C = r.shape
            assert C % N == 0
            assert T <= max_sequence_length
            assert reduce(lambda a, b: a * b, u.shape, 1) == C, "u must hold one value per channel"
            assert all(jnp.dtype(x.dtype) == jnp.dtype(r.dtype) for x in (k, v, w, u))
            return B, T, C, C // N, _code(r.dtype), _out_dtype(r.dtype)

        def fwd_call(r, k, v, w, u):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            desc = _native.create_descriptor(B, T, C, H, False, code, _code(odt))
            return jax.ffi.ffi_call("wkv_forward", jax.ShapeDtypeStruct(r.shape, odt),
                                    custom_call_api_version=2, legacy_backend_config=desc)(r, k, v, w, u)

        def bwd_call(r, k, v, w, u, gy):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            desc = _native.create_descriptor(B, T, C, H, False, code, _code(odt))
            ws = max(int(lib.wkv6_backward_workspace_bytes(code, B, T, C, H)), 16)
            big = jax.ShapeDtypeStruct(r.shape, odt)
            outs = jax.ffi.ffi_call(
                "wkv_backward",
                (big, big, big, big, jax.ShapeDtypeStruct((B,) + tuple(u.shape), odt),
                 jax.ShapeDtypeStruct((ws,), jnp.uint8)),
                custom_call_api_version=2, legacy_backend_config=desc)(r, k, v, w, u, gy.astype(odt))
            gr, gk, gv, gw, gu, _ = outs
            return gr, gk, gv, gw, jnp.sum(gu, axis=0)

        def saved_bytes(r, k, v, w, u):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            return int(lib.wkv6_saved_bytes(code, _native.ALGO_AUTO, B, T, C, H))

        def fwd_save_call(r, k, v, w, u, nsave):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            desc = _native.create_descriptor(B, T, C, H, False, code, _code(odt))
            return jax.ffi.ffi_call("wkv_forward_save",
                                    (jax.ShapeDtypeStruct(r.shape, odt), jax.ShapeDtypeStruct((nsave,), jnp.uint8)),
                                    custom_call_api_version=2, legacy_backend_config=desc)(r, k, v, w, u)

        def bwd_saved_call(r, k, v, w, u, gy, saved):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            desc = _native.create_descriptor(B, T, C, H, False, code, _code(odt))
            big = jax.ShapeDtypeStruct(r.shape, odt)
            # the call works inside the saved block: it is handed on as a result that aliases the operand
            outs = jax.ffi.ffi_call(
                "wkv_backward_saved",
                (big, big, big, big, jax.ShapeDtypeStruct((B,) + tuple(u.shape), odt),
                 jax.ShapeDtypeStruct(saved.shape, jnp.uint8), jax.ShapeDtypeStruct(tuple(u.shape), odt)),
                custom_call_api_version=2, legacy_backend_config=desc,
                input_output_aliases={6: 5})(r, k, v, w, u, gy.astype(odt), saved)
            gr, gk, gv, gw, _, _, gu_sum = outs
            return gr, gk, gv, gw, gu_sum

        @jax.custom_vjp
        def rwkv_normal_operator(r, k, v, w, u):
            return fwd_call(r, k, v, w, u)

        def vjp_fwd(r, k, v, w, u):
            nsave = saved_bytes(r, k, v, w, u)
            if nsave > 0:
                y, saved = fwd_save_call(r, k, v, w, u, nsave)
                return y, (r, k, v, w, u, saved)
            return fwd_call(r, k, v, w, u), (r, k, v, w, u, None)

        def vjp_bwd(res, gy):
            r, k, v, w, u, saved = res
            if saved is not None:
                gr, gk, gv, gw, gu = bwd_saved_call(r, k, v, w, u, gy, saved)
            else:
                gr, gk, gv, gw, gu = bwd_call(r, k, v, w, u, gy)
            dt = r.dtype
            return gr.astype(dt), gk.astype(dt), gv.astype(dt), gw.astype(dt), gu.astype(dt).reshape(u.shape)

        rwkv_normal_operator.defvjp(vjp_fwd, vjp_bwd)
        self.rwkv_normal_operator = rwkv_normal_operator

        def rwkv_fwd_with_state(r, k, v, w, u, init_state=None, state_map=None):
            B, T, C, H, code, odt = check(r, k, v, w, u)
            y_t = jax.ShapeDtypeStruct(r.shape, odt)
            s_t = jax.ShapeDtypeStruct((B, H, N, N), odt)
            if init_state is None:
                assert state_map is None, "state_map needs init_state"
                desc = _native.create_descriptor(B, T, C, H, False, code, _code(odt))
                return jax.ffi.ffi_call("wkv_forward_with_state", (y_t, s_t), custom_call_api_version=2,
                                        legacy_backend_config=desc)(r, k, v, w, u)
            assert init_state.ndim in (3, 4), "init_state must be (state_kinds, H, N, N) or (H, N, N)"
            if init_state.ndim == 3:
                init_state = init_state[None]
            kinds = init_state.shape[0]
            assert tuple(init_state.shape[1:]) == (H, N, N) and kinds <= B
            assert jnp.dtype(init_state.dtype) == odt, "init_state dtype must be %s" % odt
            if state_map is None:
                if kinds == 1:
                    state_map = np.zeros((B,), np.int64)
                elif kinds == B:
                    state_map = np.arange(B, dtype=np.int64)
                else:
                    raise ValueError("state_map cannot be inferred from init_state; pass it explicitly")
            if isinstance(state_map, (list, tuple)):
                state_map = np.asarray(state_map, np.int64)
            assert jnp.dtype(state_map.dtype) in (jnp.dtype("int32"), jnp.dtype("int64"))
            assert tuple(state_map.shape) == (B,), "state_map must have shape (batch,)"
            if isinstance(state_map, np.ndarray):
                assert (state_map >= 0).all() and (state_map < kinds).all(), \
                    "state_map values must lie in [0, %d)" % kinds
            # the kernel reads 64-bit indices; without jax_enable_x64 an int64 array cannot exist on
            # the device, so the map is shipped as pairs of int32 (little endian: value, 0)
            m32 = jnp.asarray(state_map).astype(jnp.int32)
            m64 = jnp.stack([m32, jnp.zeros_like(m32)], axis=-1).reshape(2 * B)
            desc = _native.create_descriptor(B, T, C, H, True, code, _code(odt))
            return jax.ffi.ffi_call("wkv_forward_with_state", (y_t, s_t), custom_call_api_version=2,
                                    legacy_backend_config=desc)(m64, r, k, v, w, u, init_state)

        self.rwkv_fwd_with_state = rwkv_fwd_with_state

    def __call__(self, r, k, v, w, u, return_state=False, init_state=None, state_map=None):
        if hasattr(u, "value"):
            u = u.value
        if return_state:
            return self.rwkv_fwd_with_state(r, k, v, w, u, init_state, state_map)
        return self.rwkv_normal_operator(r, k, v, w, u), None
