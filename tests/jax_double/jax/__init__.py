"""A TEST DOUBLE for jax -- not jax, and never importable outside the one test that puts this folder
on sys.path.  jax is not installed in this image, so rwkv_kernel/jax_rwkv_kernel.py could never
execute; this package stands in for exactly the entry points that module touches, so that its own
logic (descriptor, buffer order of the three custom-call targets, the extra scratch result, dtype
rules, batch sum of gu, packing of state_map, custom_vjp wiring) runs against the REAL targets of
libwkv6_gfx950.so on the GPU:

    jax.ShapeDtypeStruct, jax.custom_vjp (+ defvjp), jax.vjp for such a function,
    jax.ffi.pycapsule / register_ffi_target / ffi_call  (jax/ffi.py),
    jax.numpy: dtype, the dtype names, asarray, stack, zeros_like, sum  (jax/numpy.py).

Arrays are torch tensors on the current CUDA device (with an `astype` method).  ffi_call does what
XLA's legacy (api_version 0) custom call does: operands then results in one array of device
pointers, the opaque descriptor and its length, the stream.  What it cannot show is that real jax
traces, lowers and differentiates the module the same way.
"""
import torch

from . import ffi, numpy  # noqa: F401


class Array(torch.Tensor):
    def astype(self, dtype):
        return self.to(numpy.dtype(dtype)).as_subclass(Array)


def _wrap(t):
    return t.as_subclass(Array)


class ShapeDtypeStruct:
    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(int(d) for d in shape), numpy.dtype(dtype)


class custom_vjp:
    """f with a hand-written derivative: calling it runs f; jax.vjp(f, ...) runs the two rules."""

    def __init__(self, fun):
        self.fun, self.fwd, self.bwd = fun, None, None

    def defvjp(self, fwd, bwd):
        self.fwd, self.bwd = fwd, bwd

    def __call__(self, *args):
        return self.fun(*args)


def vjp(fun, *primals):
    assert isinstance(fun, custom_vjp) and fun.fwd is not None, "the double differentiates custom_vjp functions only"
    out, residuals = fun.fwd(*primals)
    return out, lambda cotangent: tuple(fun.bwd(residuals, cotangent))
