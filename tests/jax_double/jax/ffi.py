"""jax.ffi of the test double (see the package docstring)."""
import ctypes

import torch

_TARGETS = {}


def pycapsule(fn):
    assert isinstance(fn, ctypes._CFuncPtr), "expects the ctypes function object of a library symbol"
    return fn


def register_ffi_target(name, capsule, platform, api_version):
    assert platform == "ROCM" and api_version == 0, (platform, api_version)
    capsule.restype = None
    capsule.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_char_p, ctypes.c_size_t]
    _TARGETS[name] = capsule


def ffi_call(name, result_shape_dtypes, custom_call_api_version, legacy_backend_config, input_output_aliases=None):
    """Returns the callable that runs target `name` the way XLA's legacy custom call does."""
    from . import ShapeDtypeStruct, _wrap
    assert custom_call_api_version == 2, "API_VERSION_STATUS_RETURNING_UNIFIED carries the opaque string"
    single = isinstance(result_shape_dtypes, ShapeDtypeStruct)
    specs = [result_shape_dtypes] if single else list(result_shape_dtypes)
    opaque = bytes(legacy_backend_config)

    def run(*operands):
        ops = [o.contiguous() for o in operands]
        assert all(o.is_cuda for o in ops)
        results = [torch.empty(s.shape, dtype=s.dtype, device=ops[0].device) for s in specs]
        # a result that aliases an operand is the operand's buffer; the operand itself must look untouched to the
        # rest of the program, so (as XLA does when the value is still needed) the call gets a copy of it
        for operand, result in (input_output_aliases or {}).items():
            assert tuple(ops[operand].shape) == tuple(specs[result].shape) and ops[operand].dtype == specs[result].dtype
            ops[operand] = ops[operand].clone()
            results[result] = ops[operand]
        bufs = ops + results
        arr = (ctypes.c_void_p * len(bufs))(*[b.data_ptr() for b in bufs])
        _TARGETS[name](torch.cuda.current_stream().cuda_stream, arr, opaque, len(opaque))
        outs = [_wrap(t) for t in results]
        return outs[0] if single else tuple(outs)

    return run
