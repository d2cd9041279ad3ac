"""ctypes binding of libwkv6_gfx950.so (the C ABI declared in include/wkv6.h).

The library is built in-tree by star-rwkv6_amd/build.py.  There is no fallback: if it is missing
or a call fails, an exception is raised.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, "lib", "libwkv6_gfx950.so")

BF16, F16, F32 = 0, 1, 2
ALGO_AUTO, ALGO_SCAN, ALGO_CHUNK = 0, 1, 2
STATIC_SCRATCH_BYTES = 64 << 20   # WKV6_STATIC_SCRATCH_BYTES

_i64, _int, _p, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); one entry per symbol include/wkv6.h declares
SIGNATURES = {
    "wkv6_status_string": (ctypes.c_char_p, [_int]),
    "wkv6_version": (_int, []),
    "wkv6_supports_head_size": (_int, [_i64]),
    "wkv6_forward": (_int, [_p, _int] + [_i64] * 4 + [_p] * 6),
    "wkv6_forward_with_state": (_int, [_p, _int] + [_i64] * 4 + [_int, _p] + [_p] * 8),
    "wkv6_forward_with_state_ex": (_int, [_p, _int, _int, _int] + [_i64] * 4 + [_int, _p] + [_p] * 8 + [_p, _sz]),
    "wkv6_forward_workspace_bytes": (_sz, [_int, _int] + [_i64] * 4),
    "wkv6_forward_gn_gate": (_int, [_p, _int, _int] + [_i64] * 4 + [_int, _p] + [_p] * 9 + [ctypes.c_float, _p, _p]),
    "wkv6_forward_gn_gate_ex": (_int, [_p, _int, _int] + [_i64] * 4 + [_int, _p] + [_p] * 9 + [ctypes.c_float, _p, _p] + [_p, _sz]),
    "wkv6_forward_gn_gate_save_supported": (_int, [_int] + [_i64] * 4),
    "wkv6_forward_gn_gate_save": (_int, [_p, _int] + [_i64] * 4 + [_p] * 8 + [ctypes.c_float] + [_p] * 4 + [_sz]),
    "wkv6_gn_gate_backward": (_int, [_p, _int] + [_i64] * 4 + [_p] * 10),
    "wkv6_shift_mix_supported": (_int, [_int, _i64, _i64]),
    "wkv6_shift_mix_x": (_int, [_p, _int] + [_i64] * 3 + [_p] * 3),
    "wkv6_shift_mix_five": (_int, [_p, _int] + [_i64] * 4 + [_p] * 9),
    "wkv6_shift_mix_five_backward": (_int, [_p, _int] + [_i64] * 4 + [_p] * 10 + [_i64, _p, _p]),
    "wkv6_shift_mix_x_backward": (_int, [_p, _int] + [_i64] * 3 + [_p] * 7),
    "wkv6_backward": (_int, [_p, _int] + [_i64] * 4 + [_p] * 11 + [_p, _sz]),
    "wkv6_backward_workspace_bytes": (_sz, [_int] + [_i64] * 4),
    "wkv6_backward_static": (_int, [_p, _int] + [_i64] * 4 + [_p] * 11),
    "wkv6_forward_ex": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 6 + [_p, _sz]),
    "wkv6_backward_ex": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 11 + [_p, _sz]),
    "wkv6_backward_workspace_bytes_ex": (_sz, [_int, _int] + [_i64] * 4),
    "wkv6_backward_with_state_workspace_bytes": (_sz, [_int, _int] + [_i64] * 4),
    "wkv6_backward_with_state": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 14 + [_p, _sz]),
    "wkv6_saved_bytes": (_sz, [_int, _int] + [_i64] * 4),
    "wkv6_forward_save": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 6 + [_p, _sz]),
    "wkv6_backward_saved": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 11 + [_p, _sz]),
    "wkv6_backward_saved_sum": (_int, [_p, _int, _int] + [_i64] * 4 + [_p] * 12 + [_p, _sz]),
    "wkv6_create_descriptor": (_sz, [_int] * 7 + [_p]),
    "wkv_forward": (None, [_p, ctypes.POINTER(_p), ctypes.c_char_p, _sz]),
    "wkv_backward": (None, [_p, ctypes.POINTER(_p), ctypes.c_char_p, _sz]),
    "wkv_forward_with_state": (None, [_p, ctypes.POINTER(_p), ctypes.c_char_p, _sz]),
    "wkv_forward_save": (None, [_p, ctypes.POINTER(_p), ctypes.c_char_p, _sz]),
    "wkv_backward_saved": (None, [_p, ctypes.POINTER(_p), ctypes.c_char_p, _sz]),
    "wkv6_last_status": (_int, []),
    "wkv6_last_hip_error": (_int, []),
}

_lib = None


class WKV6Error(RuntimeError):
    pass


def load():
    """Returns the loaded library; raises WKV6Error when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise WKV6Error(
                "%s not found: build it with `python star-rwkv6_amd/build.py` (hipcc, gfx950). "
                "There is no CPU fallback for the torch/jax flavours." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        lib = load()
        msg = lib.wkv6_status_string(status).decode()
        if status == 4:
            msg += " (hipError %d)" % lib.wkv6_last_hip_error()
        raise WKV6Error("wkv6: " + msg)


def create_descriptor(B, T, C, H, S, x_type, y_type):
    """28-byte opaque descriptor of the XLA custom-call targets."""
    buf = ctypes.create_string_buffer(28)
    n = load().wkv6_create_descriptor(B, T, C, H, int(bool(S)), x_type, y_type, buf)
    return buf.raw[:n]
