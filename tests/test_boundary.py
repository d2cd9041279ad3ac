"""The Python surface mirrors the reference's rwkv_kernel package (names, signature, errors).
CPU only: the portable flavour is compared with the oracle; the torch flavour is exercised up to
its argument checks (its kernels need the GPU)."""
import importlib
import os
import sys

import numpy as np
import pytest
import torch


def _fresh_import(backend):
    os.environ["KERAS_BACKEND"] = backend
    for m in [m for m in sys.modules if m == "rwkv_kernel" or m.startswith("rwkv_kernel.")]:
        if not m.endswith("_native"):
            del sys.modules[m]
    return importlib.import_module("rwkv_kernel")


@pytest.fixture()
def restore_backend():
    old = os.environ.get("KERAS_BACKEND")
    yield
    os.environ["KERAS_BACKEND"] = old or "torch"
    _fresh_import(os.environ["KERAS_BACKEND"])


def test_backend_switch_and_exports(restore_backend):
    pkg = _fresh_import("torch")
    assert pkg.RWKVKernelOperator.__module__.endswith("torch_rwkv_kernel")
    assert pkg.OPSKernelOperator.__module__.endswith("ops_rwkv_kernal")
    pkg = _fresh_import("numpy")
    assert pkg.RWKVKernelOperator is pkg.OPSKernelOperator
    os.environ.pop("KERAS_BACKEND")
    for m in [m for m in sys.modules if m == "rwkv_kernel"]:
        del sys.modules[m]
    with pytest.raises(AssertionError):
        importlib.import_module("rwkv_kernel")   # rwkv_kernel/__init__.py:2 of the reference asserts the same


def test_jax_flavour_needs_jax(restore_backend):
    try:
        import jax  # noqa: F401
        pytest.skip("jax present")
    except ImportError:
        pass
    with pytest.raises(ImportError):
        _fresh_import("jax")


def test_ops_flavour_matches_oracle(oracle, restore_backend):
    pkg = _fresh_import("numpy")
    op = pkg.OPSKernelOperator(8, 64)
    B, T, H, N = 3, 11, 2, 8
    r, k, v, w, u, _ = oracle.make_inputs(B, T, H, N, 5)
    y, s = op(r.double(), k.double(), v.double(), w.double(), u.double())
    y_ref, s_ref = oracle.forward_c(r, k, v, w, u, N)
    np.testing.assert_allclose(y.numpy(), y_ref, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(s.numpy(), s_ref, rtol=1e-11, atol=1e-12)
    # state arguments: (H,N,N) shared state, explicit map, both spellings of the flag
    s0 = torch.randn(2, H, N, N, dtype=torch.float64)
    y1, s1 = op(r.double(), k.double(), v.double(), w.double(), u.double(), with_state=True,
                init_state=s0, state_map=[1, 0, 1])
    y1_ref, s1_ref = oracle.forward_c(r, k, v, w, u, N, s0.numpy(), [1, 0, 1])
    np.testing.assert_allclose(y1.numpy(), y1_ref, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(s1.numpy(), s1_ref, rtol=1e-11, atol=1e-12)
    y2, _ = op(r.double(), k.double(), v.double(), w.double(), u.double(), return_state=True, init_state=s0[0])
    np.testing.assert_allclose(y2.numpy(), oracle.forward_c(r, k, v, w, u, N, s0.numpy()[:1], [0] * B)[0],
                               rtol=1e-11, atol=1e-12)
    with pytest.raises(ValueError):      # 2 states for 3 rows: map cannot be inferred (ops_rwkv_kernal.py:58)
        op(r, k, v, w, u, init_state=s0.float())
    with pytest.raises(AssertionError):  # out-of-range map
        op(r, k, v, w, u, init_state=s0.float(), state_map=[0, 2, 0])
    with pytest.raises(AssertionError):  # C not a multiple of head size
        pkg.OPSKernelOperator(7, 64)(r, k, v, w, u)


def test_torch_flavour_argument_checks(restore_backend):
    pkg = _fresh_import("torch")
    with pytest.raises(Exception):
        pkg.RWKVKernelOperator(132, 64)         # the library has kernels for the multiples of 4 up to 128
    assert pkg.RWKVKernelOperator(32, 64).head_size == 32 and pkg.RWKVKernelOperator(12, 64).head_size == 12
    with pytest.raises(AssertionError):
        pkg.RWKVKernelOperator(6, 64)           # head size must be a multiple of 4 (rwkv_kernels.cu:101)
    op = pkg.RWKVKernelOperator(64, 1024)
    assert op.head_size == 64 and op.max_sequence_length == 1024
    x = torch.zeros(2, 4, 128)
    u = torch.zeros(2, 64)
    with pytest.raises(AssertionError):
        op(x, x, x, x, u)                       # tensors must live on the GPU (torch_rwkv_kernel.py:107-111)
    with pytest.raises(AssertionError):
        op(torch.zeros(2, 4, 100), x, x, x, u)  # C % head_size


class _Var:
    def __init__(self, value):
        self.value = value


def test_u_may_be_a_framework_variable(restore_backend):
    # rwkv6_model.py passes a Keras variable; .value is unwrapped (torch_rwkv_kernel.py:104-105)
    pkg = _fresh_import("numpy")
    op = pkg.OPSKernelOperator(4, 8)
    r = torch.randn(1, 3, 8)
    u = torch.randn(2, 4)
    a, _ = op(r, r, r, r, u)
    b, _ = op(r, r, r, r, _Var(u))
    assert torch.equal(a, b)
