"""Head sizes other than 64 (the reference builds for any multiple of 4, rwkv_kernel/torch_rwkv_kernel.py:13; its own
scripts run 8 -- rwkv_kernel/jax_rwkv_kernel.py:513-518 -- and 32 -- deprecated_code/test_rwkv_torch.py:62-99):
the plain calls of the operator class through the C ABI against the float64 oracle."""
import numpy as np
import pytest
import torch

from _util import cast_inputs, check_close, out_dtype, to_np

pytestmark = pytest.mark.gpu

DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _op(N):
    assert torch.cuda.is_available(), "these tests need the GPU"
    import rwkv_kernel

    return rwkv_kernel.RWKVKernelOperator(N, 4096)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("N,B,T,H", [(8, 2, 37, 3), (8, 1, 16, 9), (16, 3, 50, 2), (32, 2, 64, 4), (32, 1, 129, 1), (32, 2, 5, 3),
                                     # head sizes that do not divide the workgroup: 5 heads of 12 per workgroup, 3 of 20, 2 of 24, one of 40 ...
                                     (4, 2, 19, 35), (12, 2, 33, 7), (20, 1, 40, 4), (24, 2, 21, 3), (40, 2, 18, 2), (48, 1, 35, 3),
                                     (60, 1, 17, 2), (96, 1, 34, 2), (128, 2, 20, 1)])
def test_forward_backward(oracle, dt, N, B, T, H):
    dtype = DTYPES[dt]
    odt = out_dtype(dtype)
    op = _op(N)
    ins = oracle.make_inputs(B, T, H, N, 7 * N + T)
    dev, ref = cast_inputs(ins[:5], dtype)
    gyd, gyr = cast_inputs(ins[5:6], odt)
    leaves = [x.clone().requires_grad_(True) for x in dev]
    y, none = op(*leaves)
    assert none is None and y.dtype == odt
    y.backward(gyd[0])
    torch.cuda.synchronize()
    check_close("y", y, oracle.forward_c(*ref, N)[0], odt)
    for name, x, want in zip("gr gk gv gw gu".split(), leaves, oracle.backward_c(*ref, gyr[0], N)):
        check_close(name, to_np(x.grad).reshape(want.shape), want, odt, is_grad=True)
    gw = leaves[3].grad
    assert float(gw[:, 0].abs().max()) == 0.0 and float(gw[:, -1].abs().max()) == 0.0


def test_reference_script_shape_head_size_8(oracle):
    # rwkv_kernel/jax_rwkv_kernel.py:513-518: B=2 T=32 C=16 H=2 (N = 8), constant inputs r=k=v=u=1, w=-4:
    # y_t = N (1 + (1 - d^t) / (1 - d)), d = exp(-exp(-4))
    B, T, H, N = 2, 32, 2, 8
    op = _op(N)
    one = torch.ones(B, T, H * N, device="cuda")
    with torch.no_grad():
        y, _ = op(one, one, one, one * 0 - 4, torch.ones(H * N, device="cuda"))
    d = np.exp(-np.exp(-4.0))
    np.testing.assert_allclose(to_np(y)[1, :, 5], N * (1 + (1 - d ** np.arange(T)) / (1 - d)), rtol=2e-6)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("N", [8, 32, 12, 48, 128])
def test_state_in_and_out_with_map(oracle, dt, N):
    B, T, H = 4, 45, 3
    dtype = DTYPES[dt]
    op = _op(N)
    ins = oracle.make_inputs(B, T, H, N, 11, with_state=True)
    dev, ref = cast_inputs(ins[:5], dtype)
    s_dev, s_ref = cast_inputs([ins[6][:2]], torch.float32)
    smap = [1, 0, 0, 1]
    with torch.no_grad():
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
    torch.cuda.synchronize()
    y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
    check_close("y", y, y_ref, out_dtype(dtype))
    check_close("sT", sT, sT_ref, out_dtype(dtype), is_grad=True)


@pytest.mark.parametrize("N", [8, 16, 32, 4, 20, 56, 100])
def test_gradients_through_the_state(oracle, N):
    B, T, H = 2, 41, 2
    op = _op(N)
    ins = oracle.make_inputs(B, T, H, N, 13, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.float32)
    gyd, gyr = cast_inputs(ins[5:6], torch.float32)
    s0 = ins[6].float() * 3
    gS = torch.randn(B, H, N, N, generator=torch.Generator().manual_seed(N))
    leaves = [x.clone().requires_grad_(True) for x in dev]
    s0_dev = s0.cuda().requires_grad_(True)
    y, sT = op(*leaves, return_state=True, init_state=s0_dev)
    loss = (y * gyd[0]).sum() + (sT * gS.cuda()).sum()
    got = torch.autograd.grad(loss, leaves + [s0_dev])
    torch.cuda.synchronize()
    want = oracle.backward_state_c(*ref, gyr[0], N, to_np(s0), to_np(gS))
    for name, g, gr in zip("gr gk gv gw gu gs0".split(), got, want):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.float32, is_grad=True)


def test_what_small_heads_do_not_have():
    from rwkv_kernel import _native

    lib = _native.load()
    assert lib.wkv6_supports_head_size(8) and lib.wkv6_supports_head_size(16) and lib.wkv6_supports_head_size(32) and lib.wkv6_supports_head_size(64)
    assert lib.wkv6_supports_head_size(12) and lib.wkv6_supports_head_size(128)
    assert not lib.wkv6_supports_head_size(10) and not lib.wkv6_supports_head_size(132)
    # no saved states, no chunk form, no fused stage
    assert lib.wkv6_saved_bytes(_native.BF16, _native.ALGO_AUTO, 2, 256, 64, 2) == 0
    assert lib.wkv6_backward_workspace_bytes(_native.F32, 2, 100, 64, 2) == (2 * 100 * 64 + 2 * 64) * 4
    x = torch.zeros(64, device="cuda")
    p = x.data_ptr()
    assert lib.wkv6_forward_ex(None, _native.BF16, _native.ALGO_CHUNK, 2, 256, 64, 2, *([p] * 6), None, 0) == 2
    assert lib.wkv6_forward_gn_gate_save_supported(_native.BF16, 2, 256, 64, 2) == 0
