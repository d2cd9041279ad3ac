"""CPU-side checks of the C ABI: the library loads, exports every symbol include/wkv6.h declares,
and rejects bad arguments with status codes before touching the GPU (no compute calls here)."""
import ctypes
import os
import re
import struct

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def native():
    from rwkv_kernel import _native

    if not os.path.exists(_native.LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()
    return _native


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "wkv6.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([a-z][a-z0-9_]*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(n for n in names if n.startswith("wkv")))


def test_every_declared_symbol_is_exported_and_bound(native):
    lib = native.load()
    declared = _declared_functions()
    assert len(declared) >= 18
    for name in declared:
        assert hasattr(lib, name), "missing export: " + name
        assert name in native.SIGNATURES, "ctypes binding lacks " + name
    assert sorted(native.SIGNATURES) == declared


def test_version_and_head_size(native):
    lib = native.load()
    assert lib.wkv6_version() >= 100
    assert lib.wkv6_supports_head_size(64) == 1
    assert lib.wkv6_supports_head_size(32) == 1 and lib.wkv6_supports_head_size(8) == 1   # the plain calls
    assert lib.wkv6_supports_head_size(12) == 1 and lib.wkv6_supports_head_size(128) == 1   # any multiple of 4 up to 128
    assert lib.wkv6_supports_head_size(6) == 0 and lib.wkv6_supports_head_size(132) == 0 and lib.wkv6_supports_head_size(0) == 0
    assert lib.wkv6_status_string(0) == b"ok"
    assert b"workspace" in lib.wkv6_status_string(3)


def test_descriptor_is_the_reference_28_byte_struct(native):
    # {int B,T,C,H; bool S; enum x_type,y_type}, rwkv_kernel/jax_kernel/kernels.h:32-42
    d = native.create_descriptor(8, 1024, 2048, 32, True, native.BF16, native.BF16)
    assert len(d) == 28
    B, T, C, H, S, x, y = struct.unpack("<iiiiB3xii", d)
    assert (B, T, C, H, S, x, y) == (8, 1024, 2048, 32, 1, 0, 0)
    d = native.create_descriptor(1, 16, 8, 1, False, native.F16, native.F32)
    assert struct.unpack("<iiiiB3xii", d)[4:] == (0, 1, 2)


def test_argument_validation_returns_status_codes(native):
    lib = native.load()
    fake = 0x1000  # never dereferenced: validation fails first
    args = [fake] * 6
    assert lib.wkv6_forward(None, native.BF16, 2, 16, 128, 2, None, *args[1:]) == 1        # null pointer
    assert lib.wkv6_forward(None, 7, 2, 16, 128, 2, *args) == 1                            # unknown dtype
    assert lib.wkv6_forward(None, native.BF16, 2, 16, 130, 2, *args) == 2                  # head size 65
    assert lib.wkv6_forward(None, native.BF16, 2, 16, 20, 2, *args) == 2                   # head size 10
    assert lib.wkv6_forward(None, native.BF16, 2, 16, 264, 2, *args) == 2                  # head size 132
    assert lib.wkv6_forward_gn_gate(None, native.BF16, native.BF16, 2, 16, 64, 2, 0, None, *([fake] * 6), fake, fake, fake, 1e-5, fake, None) == 2   # head size 32: plain calls only
    assert lib.wkv6_forward(None, native.BF16, 0, 16, 128, 2, *args) == 1                  # empty batch
    assert lib.wkv6_forward(None, native.BF16, 2, 16, 128, 2, fake + 2, *args[1:]) == 1    # misaligned
    assert lib.wkv6_forward_ex(None, native.F32, native.ALGO_CHUNK, 2, 63, 128, 2, *args, None, 0) == 2   # no chunk form below 64 tokens
    assert lib.wkv6_forward_ex(None, native.BF16, 3, 2, 64, 128, 2, *args, None, 0) == 1   # unknown algo
    need = lib.wkv6_backward_workspace_bytes(native.BF16, 8, 1024, 2048, 32)
    assert need == 8 * 1024 * 2048 * 4
    assert lib.wkv6_backward_workspace_bytes_ex(native.F32, native.ALGO_SCAN, 2, 100, 128, 2) == 2 * 100 * 128 * 4
    assert lib.wkv6_backward_workspace_bytes_ex(native.F32, native.ALGO_AUTO, 2, 100, 128, 2) == 2 * 2 * 4 * 64 * 64 * 4   # fp32 chunk states
    assert lib.wkv6_backward_workspace_bytes_ex(native.F16, native.ALGO_AUTO, 2, 40, 128, 2) == 2 * 40 * 128 * 4
    assert lib.wkv6_backward_workspace_bytes_ex(native.BF16, native.ALGO_CHUNK, 2, 100, 128, 2) == 2 * 128 * 128 * 4
    assert lib.wkv6_backward_workspace_bytes(native.BF16, 2, 16, 130, 2) == 0
    gargs = [fake] * 11
    assert lib.wkv6_backward(None, native.BF16, 2, 16, 128, 2, *gargs, None, 0) == 3       # workspace missing
    assert lib.wkv6_backward(None, native.BF16, 2, 16, 128, 2, *gargs, fake, 16) == 3      # workspace too small
    assert lib.wkv6_forward_with_state(None, native.BF16, 2, 16, 128, 2, 1, None, *args[:5], None, fake, fake) == 1


def test_misaligned_pointers_are_refused_by_the_fused_entry_points(native):
    """The token-shift, low-rank-mixer and group-norm entry points use 16-byte vector accesses on every
    tensor argument: a pointer off a 16-byte boundary is WKV6_ERR_ARG before anything is launched, as in
    the operator's own entry points; so is a negative or NaN epsilon."""
    lib = native.load()
    ok, off = 0x10000, 0x10008
    B, T, C, R, H = 2, 64, 128, 32, 2

    def variants(n):
        for i in range(n):
            yield [off if j == i else ok for j in range(n)]

    for a in variants(3):
        assert lib.wkv6_shift_mix_x(None, native.BF16, B, T, C, *a) == 1, a
    for a in variants(9):
        assert lib.wkv6_shift_mix_five(None, native.BF16, B, T, C, R, *a) == 1, a
    for a in variants(12):
        assert lib.wkv6_shift_mix_five_backward(None, native.BF16, B, T, C, R, *a[:10], B * T * C, *a[10:]) == 1, a
    for a in variants(7):
        assert lib.wkv6_shift_mix_x_backward(None, native.BF16, B, T, C, *a) == 1, a
    for a in variants(10):
        assert lib.wkv6_gn_gate_backward(None, native.BF16, B, T, C, H, *a) == 1, a
    saved = lib.wkv6_saved_bytes(native.BF16, native.ALGO_CHUNK, B, T, C, H)
    for eps in (-1.0, float("nan")):
        assert lib.wkv6_forward_gn_gate_save(None, native.BF16, B, T, C, H, *([ok] * 8), eps, ok, ok, ok, ok, saved) == 1, eps


def test_custom_call_rejects_bad_opaque_without_throwing(native):
    lib = native.load()
    arr = (ctypes.c_void_p * 12)(*([0x1000] * 12))
    lib.wkv_forward(None, arr, b"x" * 27, 27)
    assert lib.wkv6_last_status() == 1
    lib.wkv_backward(None, arr, None, 0)
    assert lib.wkv6_last_status() == 1
    lib.wkv_forward_save(None, arr, b"x" * 29, 29)
    assert lib.wkv6_last_status() == 1
    lib.wkv_backward_saved(None, None, b"x" * 28, 28)
    assert lib.wkv6_last_status() == 1
    # output type that contradicts the dtype rule (bf16 in -> f32 out) is refused
    bad = native.create_descriptor(1, 16, 64, 1, False, native.BF16, native.F32)
    lib.wkv_forward_with_state(None, arr, bad, len(bad))
    assert lib.wkv6_last_status() == 1


def test_missing_library_fails_loudly(native, monkeypatch):
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIB_PATH", "/nonexistent/libwkv6_gfx950.so")
    with pytest.raises(native.WKV6Error):
        native.load()
