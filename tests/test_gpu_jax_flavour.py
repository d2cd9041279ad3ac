"""rwkv_kernel/jax_rwkv_kernel.py executed on the GPU against a TEST DOUBLE of jax.

jax itself is not installed here, so this does not show that jax traces, lowers or differentiates the
module; it shows that the module's own code -- the 28-byte descriptor, the operand and result order
of the three custom-call targets, the scratch result of the backward, the dtype rules, the batch sum
of gu, the int32-pair packing of state_map, the custom_vjp rules -- drives the REAL targets of
libwkv6_gfx950.so to the oracle's results.  The double (tests/jax_double/) hands the registered
symbols operands and results the way XLA's legacy custom call does: one array of device pointers,
the opaque descriptor, the stream."""
import importlib
import os
import sys

import numpy as np
import pytest
import torch

from _util import cast_inputs, check_close, to_np

pytestmark = pytest.mark.gpu
DOUBLE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "jax_double")


@pytest.fixture
def flavour():
    """(module rwkv_kernel.jax_rwkv_kernel imported over the double, the double's jax)."""
    assert torch.cuda.is_available(), "these tests need the GPU"
    try:
        import jax  # noqa: F401
        pytest.skip("a real jax is installed: the double is not used")
    except ImportError:
        pass
    sys.path.insert(0, DOUBLE)
    try:
        jax = importlib.import_module("jax")
        assert jax.__file__.startswith(DOUBLE)
        import rwkv_kernel  # noqa: F401  (the package; its jax flavour is imported by name below)
        mod = importlib.import_module("rwkv_kernel.jax_rwkv_kernel")
        yield mod, jax
    finally:
        sys.path.remove(DOUBLE)
        for name in [m for m in sys.modules if m == "jax" or m.startswith("jax.") or m == "rwkv_kernel.jax_rwkv_kernel"]:
            del sys.modules[name]


@pytest.mark.parametrize("B,T,H,dtype", [(2, 256, 2, torch.bfloat16), (3, 100, 1, torch.bfloat16),
                                         (2, 40, 2, torch.float32), (2, 40, 1, torch.float16),
                                         # (the differentiated call of the first two runs the saving pair's targets; so do these)
                                         (2, 128, 2, torch.float32), (1, 100, 2, torch.float16), (1, 2048, 2, torch.bfloat16)])
def test_stateless_call_and_its_vjp(flavour, oracle, B, T, H, dtype):
    mod, jax = flavour
    jnp = jax.numpy
    N = 64
    print("jax flavour over the double: B%d T%d H%d %s" % (B, T, H, dtype), flush=True)
    op = mod.RWKVKernelOperator(N, 4096)
    ins = oracle.make_inputs(B, T, H, N, 31 + T)
    dev, ref = cast_inputs(ins[:5], dtype)
    odt = torch.float32 if dtype == torch.float16 else dtype
    gyd, gyr = cast_inputs(ins[5:6], odt)
    args = [jnp.asarray(x) for x in dev]
    y, state = op(*args)
    assert state is None and y.dtype == odt and tuple(y.shape) == (B, T, H * N)
    torch.cuda.synchronize()
    y_ref, _ = oracle.forward_c(*ref, N)
    check_close("y", y, y_ref, odt)
    y2, pull = jax.vjp(op.rwkv_normal_operator, *args)
    grads = pull(jnp.asarray(gyd[0]))
    torch.cuda.synchronize()
    assert torch.equal(y2, y)
    g_ref = oracle.backward_c(*ref, gyr[0], N)
    for name, g, want in zip("gr gk gv gw".split(), grads[:4], g_ref[:4]):
        assert g.dtype == dtype and tuple(g.shape) == (B, T, H * N)      # cast back to the inputs' type (reference :166)
        check_close(name, g, want, dtype, is_grad=True)
    gu = grads[4]
    assert tuple(gu.shape) == tuple(dev[4].shape) and gu.dtype == dtype       # summed over the batch, u's shape
    check_close("gu", to_np(gu).reshape(H, N), g_ref[4], dtype, is_grad=True)
    again = pull(jnp.asarray(gyd[0]))                                          # the residuals serve a second pull
    torch.cuda.synchronize()
    for a, b in zip(grads, again):
        assert torch.equal(a, b)


def test_stateful_call_packs_the_state_map(flavour, oracle):
    mod, jax = flavour
    jnp = jax.numpy
    B, T, H, N = 4, 96, 2, 64
    op = mod.RWKVKernelOperator(N, 128)
    ins = oracle.make_inputs(B, T, H, N, 9, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    args = [jnp.asarray(x) for x in dev]
    s0 = jnp.asarray(ins[6][:3].to(torch.bfloat16).cuda())           # three kinds of initial state for four rows
    for state_map in ([2, 0, 2, 1], np.array([1, 1, 0, 2], np.int32), np.array([0, 2, 1, 0], np.int64)):
        y, ys = op(*args, return_state=True, init_state=s0, state_map=state_map)
        torch.cuda.synchronize()
        y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s0), np.asarray(state_map, np.int64))
        check_close("y", y, y_ref, torch.bfloat16)
        check_close("ys", ys, s_ref, torch.bfloat16)
        assert tuple(ys.shape) == (B, H, N, N) and ys.dtype == torch.bfloat16
    # one state for all rows ((H,N,N) or (1,H,N,N)) and one per row need no map
    y, ys = op(*args, return_state=True, init_state=s0[1])
    torch.cuda.synchronize()
    y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s0[1:2]), np.zeros(B, np.int64))
    check_close("y one state", y, y_ref, torch.bfloat16)
    check_close("ys one state", ys, s_ref, torch.bfloat16)
    s4 = jnp.asarray(ins[6].to(torch.bfloat16).cuda())
    y, ys = op(*args, return_state=True, init_state=s4)
    torch.cuda.synchronize()
    y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s4), np.arange(B))
    check_close("y per-row states", y, y_ref, torch.bfloat16)
    check_close("ys per-row states", ys, s_ref, torch.bfloat16)
    # no initial state: zero state, final state returned
    y, ys = op(*args, return_state=True)
    torch.cuda.synchronize()
    y_ref, s_ref = oracle.forward_c(*ref, N)
    check_close("y zero state", y, y_ref, torch.bfloat16)
    check_close("ys zero state", ys, s_ref, torch.bfloat16)


def test_argument_checks(flavour, oracle):
    mod, jax = flavour
    jnp = jax.numpy
    N = 64
    op = mod.RWKVKernelOperator(N, 32)
    ins = oracle.make_inputs(1, 33, 1, N, 1)
    dev, _ = cast_inputs(ins[:5], torch.float32)
    args = [jnp.asarray(x) for x in dev]
    with pytest.raises(AssertionError):
        op(*args)                                         # longer than max_sequence_length (reference :128)
    short = [a[:, :8].contiguous() for a in args[:4]] + [args[4]]
    with pytest.raises(AssertionError):
        op(short[0], short[1].astype(jnp.bfloat16), *short[2:])      # mixed dtypes
    with pytest.raises(ValueError):
        op(*[jnp.asarray(torch.cat([x, x, x])) for x in short[:4]], short[4], return_state=True,
           init_state=jnp.asarray(torch.zeros(2, 1, N, N, device="cuda")))   # 2 states for 3 rows: map needed
    with pytest.raises(Exception):
        mod.RWKVKernelOperator(132, 16)                   # head size the library is not built for (multiples of 4 up to 128)
