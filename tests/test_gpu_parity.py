"""GPU parity tests: the HIP path, called through the C ABI, against the float64 CPU oracle on
the same seeded (and identically rounded) inputs.  Run on the MI355X box with -m gpu."""
import ctypes

import numpy as np
import pytest
import torch

from _util import cast_inputs, check_close, out_dtype, to_np

pytestmark = pytest.mark.gpu

SCAN, CHUNK = 1, 2
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


@pytest.fixture(scope="module")
def op():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import rwkv_kernel

    return rwkv_kernel.RWKVKernelOperator(64, 4096)


def _run_fwd_bwd(op, dev, algo):
    op.algo = algo
    leaves = [x.clone().requires_grad_(True) for x in dev[:5]]
    y, none = op(*leaves)
    assert none is None
    y.backward(dev[5])
    torch.cuda.synchronize()
    return y, [x.grad for x in leaves]


def _case(op, oracle, B, T, H, seed, dtype, algo, strict=False, tol=None):
    # tol: the dtype whose tolerance applies (default: the output dtype).  fp16 tensors on the chunked
    # kernels produce fp32 outputs at bf16 operand precision: they are held to the 1e-2 bound.
    N = 64
    print("case B=%d T=%d H=%d seed=%d dtype=%s algo=%d" % (B, T, H, seed, dtype, algo), flush=True)
    ins = oracle.make_inputs(B, T, H, N, seed)
    odt = out_dtype(dtype)
    dev, ref = cast_inputs(ins[:5], dtype)
    gy_dev, gy_ref = cast_inputs(ins[5:6], odt)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, algo)
    assert y.dtype == odt and all(g.dtype == dtype for g in grads)
    y_ref, _ = oracle.forward_c(*ref, N)
    g_ref = oracle.backward_c(*ref, gy_ref[0], N)
    if strict:
        assert np.abs(to_np(y) - y_ref).max() <= 1e-4
    check_close("y", y, y_ref, tol or odt)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, g_ref):
        check_close(name, to_np(g).reshape(gr.shape), gr, tol or odt, is_grad=True)
    return y, grads


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_config1_forward_fp32(op, oracle, seed):
    # the fp32 correctness shape: B=2 T=128 H=4 N=64; max-abs(y) <= 1e-4
    _case(op, oracle, 2, 128, 4, seed, torch.float32, SCAN, strict=True)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("T", [1, 2, 15, 16, 17, 33, 100])
def test_scan_fwd_bwd_ragged_T(op, oracle, dt, T):
    _case(op, oracle, 2, T, 2, 10 + T, DTYPES[dt], SCAN)


def test_scan_longer_sequence_bf16(op, oracle):
    _case(op, oracle, 1, 1024, 2, 5, torch.bfloat16, SCAN)


def test_scan_longer_sequence_f32(op, oracle):
    _case(op, oracle, 1, 1024, 2, 6, torch.float32, SCAN)


def test_constant_inputs_closed_form(op):
    # reference test_jax.py:12-16: r=k=v=u=1, w=-4 -> y_t = 64*(1 + (1-d^t)/(1-d))
    B, T, C = 4, 512, 512
    one = torch.ones(B, T, C, device="cuda")
    y, _ = op(one, one, one, one * 0 - 4, torch.ones(C, device="cuda"))
    d = np.exp(-np.exp(-4.0))
    expect = 64 * (1 + (1 - d ** np.arange(T)) / (1 - d))
    got = to_np(y)
    assert got[0, 0, 0] == 64.0 and got[0, 1, 0] == 128.0
    np.testing.assert_allclose(got[2, :, 77], expect, rtol=2e-5)


def test_padding_decay_value_is_finite(op, oracle):
    # rwkv6_model.py:149-152 masks tokens with k=0, w=-1e9 (decay exactly 1)
    B, T, H = 1, 40, 1
    ins = oracle.make_inputs(B, T, H, 64, 3)
    ins[3][:, 10:20] = -1e9
    ins[1][:, 10:20] = 0
    ins[3][:, 30] = 20.0  # decay exactly 0
    dev, ref = cast_inputs(ins[:5], torch.float32)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.float32)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, SCAN)
    check_close("y", y, oracle.forward_c(*ref, 64)[0], torch.float32)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], 64)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.float32, is_grad=True)


@pytest.mark.parametrize("T", [37, 1])   # T = 1 takes the single-timestep kernel
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
def test_state_in_out(op, oracle, dt, T):
    dtype = DTYPES[dt]
    odt = out_dtype(dtype)
    B, H, N = 3, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 21, with_state=True)
    dev, ref = cast_inputs(ins[:5], dtype)
    s_dev, s_ref = cast_inputs([ins[6][:2]], odt)
    smap = [1, 0, 1]
    y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
    torch.cuda.synchronize()
    assert sT.shape == (B, H, N, N) and sT.dtype == odt and y.dtype == odt
    y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
    check_close("y", y, y_ref, odt)
    check_close("sT", sT, sT_ref, odt)
    # zero-state stateful call equals the stateless call
    y0, s0T = op(*dev, return_state=True)
    y1, none = op(*dev)
    assert none is None and torch.equal(y0, y1)
    check_close("sT0", s0T, oracle.forward_c(*ref, N)[1], odt)
    # shared single state: default map is all zeros; (H,N,N) accepted
    y2, _ = op(*dev, return_state=True, init_state=s_dev[0][0])
    check_close("y_shared", y2, oracle.forward_c(*ref, N, s_ref[0][:1], [0] * B)[0], odt)
    # activations in bf16 with the carried state in fp32, five pairs (not a multiple of the four per workgroup)
    if dt == "bf16":
        s32 = ins[6][:B].float()
        y3, s3 = op(*dev, return_state=True, init_state=s32.cuda())
        y3_ref, s3_ref = oracle.forward_c(*ref, N, to_np(s32))
        assert s3.dtype == torch.float32
        check_close("y_f32state", y3, y3_ref, odt)
        check_close("sT_f32state", s3, s3_ref, odt)


def test_state_split_consistency_fp32(op, oracle):
    # op(T1+T2) == op(T1) -> op(T2, init_state): bit-identical in fp32 state
    B, T, H, N = 2, 96, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 22)
    dev, _ = cast_inputs(ins[:5], torch.float32)
    y, sT = op(*dev, return_state=True)
    cut = 41
    a = [x[:, :cut].contiguous() for x in dev[:4]] + [dev[4]]
    b = [x[:, cut:].contiguous() for x in dev[:4]] + [dev[4]]
    ya, sa = op(*a, return_state=True)
    yb, sb = op(*b, return_state=True, init_state=sa)
    assert torch.equal(torch.cat([ya, yb], 1), y)
    assert torch.equal(sb, sT)


def test_bf16_activations_with_fp32_state(op, oracle):
    B, T, H, N = 2, 20, 1, 64
    ins = oracle.make_inputs(B, T, H, N, 23, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    s32 = ins[6].cuda()
    y, sT = op(*dev, return_state=True, init_state=s32)
    assert sT.dtype == torch.float32 and y.dtype == torch.bfloat16
    y_ref, sT_ref = oracle.forward_c(*ref, N, to_np(s32))
    check_close("y", y, y_ref, torch.bfloat16)
    assert np.abs(to_np(sT) - sT_ref).max() <= 1e-4 * max(1, np.abs(sT_ref).max())


def test_golden_fixture(op):
    import os

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "wkv6_small.npz"))
    t = {n: torch.from_numpy(z[n]).cuda() for n in "r k v w u gy s0".split()}
    op.algo = SCAN
    leaves = [t[n].clone().requires_grad_(True) for n in "r k v w u".split()]
    y, _ = op(*leaves)
    y.backward(t["gy"])
    check_close("y", y, z["y"], torch.float32)
    for n, leaf in zip("gr gk gv gw gu".split(), leaves):
        check_close(n, leaf.grad, z[n], torch.float32, is_grad=True)
    ys, sT = op(*[t[n] for n in "r k v w u".split()], return_state=True, init_state=t["s0"],
                state_map=torch.from_numpy(z["state_map"]))
    check_close("y_state", ys, z["y_state"], torch.float32)
    check_close("sT", sT, z["sT"], torch.float32)


def test_xla_custom_call_targets(op, oracle):
    # the three status-less custom-call entry points with the 28-byte descriptor
    from rwkv_kernel import _native

    lib = _native.load()
    B, T, H, N = 2, 19, 1, 64
    C = H * N
    ins = oracle.make_inputs(B, T, H, N, 31, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.float32)
    gy = ins[5].cuda()
    stream = torch.cuda.current_stream().cuda_stream

    def call(fn, bufs, desc):
        arr = (ctypes.c_void_p * len(bufs))(*[b.data_ptr() for b in bufs])
        fn(stream, arr, desc, len(desc))
        torch.cuda.synchronize()
        assert lib.wkv6_last_status() == 0

    y = torch.empty(B, T, C, device="cuda")
    call(lib.wkv_forward, dev + [y], _native.create_descriptor(B, T, C, H, False, _native.F32, _native.F32))
    y_ref, _ = oracle.forward_c(*ref, N)
    check_close("y", y, y_ref, torch.float32)

    outs = [torch.empty(B, T, C, device="cuda") for _ in range(4)] + [torch.empty(B, C, device="cuda")]
    ws = torch.empty(lib.wkv6_backward_workspace_bytes(_native.F32, B, T, C, H), dtype=torch.uint8, device="cuda")
    call(lib.wkv_backward, dev + [gy] + outs + [ws], _native.create_descriptor(B, T, C, H, False, _native.F32, _native.F32))
    g_ref = oracle.backward_c(*ref, to_np(gy), N)
    for name, g, gr in zip("gr gk gv gw".split(), outs, g_ref):
        check_close(name, g, gr, torch.float32, is_grad=True)
    check_close("gu", to_np(outs[4]).sum(0).reshape(H, N), g_ref[4], torch.float32, is_grad=True)

    s0 = ins[6].cuda()
    smap = torch.tensor([1, 0], device="cuda")
    ys = torch.empty(B, H, N, N, device="cuda")
    call(lib.wkv_forward_with_state, [smap] + dev + [s0, y, ys],
         _native.create_descriptor(B, T, C, H, True, _native.F32, _native.F32))
    y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s0), [1, 0])
    check_close("y", y, y_ref, torch.float32)
    check_close("ys", ys, s_ref, torch.float32)
    call(lib.wkv_forward_with_state, dev + [y, ys], _native.create_descriptor(B, T, C, H, False, _native.F32, _native.F32))
    check_close("ys0", ys, oracle.forward_c(*ref, N)[1], torch.float32)
    # wrong opaque length: no-op + error status, nothing thrown
    arr = (ctypes.c_void_p * 6)(*[b.data_ptr() for b in dev + [y]])
    lib.wkv_forward(stream, arr, b"x" * 27, 27)
    assert lib.wkv6_last_status() == 1


@pytest.mark.parametrize("B,T,H", [(2, 256, 2), (8, 1024, 32)])
def test_xla_custom_call_targets_bf16(op, oracle, B, T, H):
    # What a JAX caller reaches: bf16 tensors through the three custom-call targets, where the
    # library's own choice is the chunked MFMA kernels and wkv_backward has to rebuild the chunk
    # states itself; the state_map buffer is built the way the jax flavour ships it, as (value, 0)
    # int32 pairs.  At the benchmark size too.
    from rwkv_kernel import _native

    lib = _native.load()
    N = 64
    C = H * N
    print("custom-call targets bf16 B%d T%d H%d" % (B, T, H), flush=True)
    ins = oracle.make_inputs(B, T, H, N, 77, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    gyd, gyr = cast_inputs(ins[5:6], torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    bf = dict(dtype=torch.bfloat16, device="cuda")
    desc = lambda S: _native.create_descriptor(B, T, C, H, S, _native.BF16, _native.BF16)

    def call(fn, bufs, d):
        arr = (ctypes.c_void_p * len(bufs))(*[b.data_ptr() for b in bufs])
        fn(stream, arr, d, len(d))
        torch.cuda.synchronize()
        assert lib.wkv6_last_status() == 0

    y = torch.empty(B, T, C, **bf)
    call(lib.wkv_forward, dev + [y], desc(False))
    y_ref, _ = oracle.forward_c(*ref, N)
    check_close("y", y, y_ref, torch.bfloat16)

    outs = [torch.empty(B, T, C, **bf) for _ in range(4)] + [torch.empty(B, C, **bf)]
    ws = torch.empty(lib.wkv6_backward_workspace_bytes(_native.BF16, B, T, C, H), dtype=torch.uint8, device="cuda")
    call(lib.wkv_backward, dev + gyd + outs + [ws], desc(False))
    g_ref = oracle.backward_c(*ref, gyr[0], N)
    for name, g, gr in zip("gr gk gv gw".split(), outs, g_ref):
        check_close(name, g, gr, torch.bfloat16, is_grad=True)
    check_close("gu", to_np(outs[4]).sum(0).reshape(H, N), g_ref[4], torch.bfloat16, is_grad=True)

    # one state per batch row, rows permuted by the map; bf16 state = the output type
    s0 = ins[6].to(torch.bfloat16).cuda()
    perm = torch.randperm(B, generator=torch.Generator().manual_seed(3))
    m32 = perm.to(torch.int32)
    pairs = torch.stack([m32, torch.zeros_like(m32)], -1).reshape(2 * B).cuda()   # little endian int64
    ys = torch.empty(B, H, N, N, **bf)
    call(lib.wkv_forward_with_state, [pairs] + dev + [s0, y, ys], desc(True))
    y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s0), perm.numpy())
    check_close("y with state", y, y_ref, torch.bfloat16)
    check_close("ys", ys, s_ref, torch.bfloat16)
    call(lib.wkv_forward_with_state, dev + [y, ys], desc(False))
    check_close("ys from zero", ys, oracle.forward_c(*ref, N)[1], torch.bfloat16)


@pytest.mark.parametrize("B,T,H,dt", [(2, 256, 2, "bf16"), (8, 1024, 32, "bf16"), (1, 2048, 2, "bf16"), (2, 128, 2, "f32"), (2, 100, 1, "f16")])
def test_xla_custom_call_targets_of_the_saving_pair(op, oracle, B, T, H, dt):
    # The targets behind the jax flavour's custom_vjp rules: wkv_forward_save leaves y and the saved block,
    # wkv_backward_saved works inside the result that aliases the block and returns gu summed over the batch.
    # Run twice from one forward (the second time on a separate result buffer, which the target fills from the
    # operand first) and with the operand checked for being left alone.  (1, 2048, 2): the pair runs in time segments.
    from rwkv_kernel import _native

    lib = _native.load()
    N = 64
    C = H * N
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32, "f16": torch.float16}[dt]
    code = {"bf16": _native.BF16, "f32": _native.F32, "f16": _native.F16}[dt]
    odt = out_dtype(dtype)
    ocode = _native.BF16 if dt == "bf16" else _native.F32
    print("custom-call targets of the saving pair %s B%d T%d H%d" % (dt, B, T, H), flush=True)
    ins = oracle.make_inputs(B, T, H, N, 78)
    dev, ref = cast_inputs(ins[:5], dtype)
    gyd, gyr = cast_inputs(ins[5:6], odt)
    stream = torch.cuda.current_stream().cuda_stream
    desc = _native.create_descriptor(B, T, C, H, False, code, ocode)
    nsave = lib.wkv6_saved_bytes(code, _native.ALGO_AUTO, B, T, C, H)
    assert nsave > 0

    def call(fn, bufs):
        arr = (ctypes.c_void_p * len(bufs))(*[b.data_ptr() for b in bufs])
        fn(stream, arr, desc, len(desc))
        torch.cuda.synchronize()
        assert lib.wkv6_last_status() == 0

    y = torch.empty(B, T, C, dtype=odt, device="cuda")
    saved = torch.empty(nsave, dtype=torch.uint8, device="cuda")
    call(lib.wkv_forward_save, dev + [y, saved])
    check_close("y", y, oracle.forward_c(*ref, N)[0], odt)
    g_ref = oracle.backward_c(*ref, gyr[0], N)
    kept = saved.clone()
    first = None
    for aliased in (False, True):
        outs = [torch.full((B, T, C), 7.0, dtype=odt, device="cuda") for _ in range(4)] + [torch.empty(B, C, dtype=odt, device="cuda")]
        gu_sum = torch.empty(C, dtype=odt, device="cuda")
        block = saved if aliased else torch.empty_like(saved)
        call(lib.wkv_backward_saved, dev + gyd + [saved] + outs + [block, gu_sum])
        if not aliased:
            assert torch.equal(saved, kept)          # two buffers: the operand is left alone
        for name, g, want in zip("gr gk gv gw".split(), outs, g_ref):
            check_close(name, g, want, odt, is_grad=True)
        check_close("gu", to_np(gu_sum).reshape(H, N), g_ref[4], odt, is_grad=True)
        if first is None:
            first = [g.clone() for g in outs[:4]] + [gu_sum.clone()]
        else:
            for a, b in zip(first, outs[:4] + [gu_sum]):
                assert torch.equal(a, b)             # the same block, the same result


def test_xla_saving_pair_refuses_shapes_that_save_nothing(op):
    from rwkv_kernel import _native

    lib = _native.load()
    B, T, C, H = 2, 16, 64, 1                        # too short for a chunk form: nothing to save
    assert lib.wkv6_saved_bytes(_native.F32, _native.ALGO_AUTO, B, T, C, H) == 0
    desc = _native.create_descriptor(B, T, C, H, False, _native.F32, _native.F32)
    x = torch.zeros(B, T, C, device="cuda")
    arr = (ctypes.c_void_p * 14)(*([x.data_ptr()] * 14))
    lib.wkv_forward_save(None, arr, desc, len(desc))
    assert lib.wkv6_last_status() == 2
    lib.wkv_backward_saved(None, arr, desc, len(desc))
    assert lib.wkv6_last_status() == 2
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------
# chunk-parallel MFMA path (bf16 tensors)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("B,T,H", [(1, 32, 1), (2, 64, 2), (2, 100, 1), (1, 129, 3), (2, 1000, 2), (1, 2048, 1)])
def test_chunk_fwd_bwd_bf16(op, oracle, B, T, H):
    _case(op, oracle, B, T, H, 40 + T, torch.bfloat16, CHUNK)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_mixed_shape_mfma_chains_keep_both_terms(op, oracle, seed):
    """The chunked kernels chain 16x16x32 and 16x16x16 MFMAs through one accumulator (y = R~ S + A V,
    and X, W, gv in the backward).  On gfx950 a second MFMA of the other shape issued too close behind the
    first read a stale accumulator, i.e. dropped the first term; the kernels keep a fixed gap there
    (chain_gap in wkv6_mfma.h).  With almost no decay (w = -6) the state terms carry most of every
    output, so a dropped term is an error of order one -- at the smallest shapes, one workgroup, where
    nothing else perturbs the instruction timing."""
    N = 64
    for T in (64, 128, 80):
        ins = oracle.make_inputs(1, T, 1, N, 900 + seed)
        ins[3] = torch.full_like(ins[3], -6.0)
        dev, ref = cast_inputs(ins[:5], torch.bfloat16)
        gy_dev, gy_ref = cast_inputs(ins[5:6], torch.bfloat16)
        y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
        y_ref, _ = oracle.forward_c(*ref, N)
        g_ref = oracle.backward_c(*ref, gy_ref[0], N)
        check_close("y", y, y_ref, torch.bfloat16)
        for name, g, gr in zip("gr gk gv gw gu".split(), grads, g_ref):
            check_close(name, to_np(g).reshape(gr.shape), gr, torch.bfloat16, is_grad=True)


@pytest.mark.parametrize("B,T,H", [(1, 16, 1), (1, 48, 1), (2, 333, 2), (3, 1024, 4), (1, 80, 5)])
def test_chunk_more_shapes_bf16(op, oracle, B, T, H):
    # T below the AUTO threshold, T % 64 != 0 with full tiles, ragged T, odd head counts
    _case(op, oracle, B, T, H, 60 + T, torch.bfloat16, CHUNK)


def test_chunk_state_in_out(op, oracle):
    B, T, H, N = 3, 150, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 51, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    op.algo = CHUNK
    for sdt in (torch.bfloat16, torch.float32):
        s_dev, s_ref = cast_inputs([ins[6][:2]], sdt)
        smap = [1, 0, 1]
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
        torch.cuda.synchronize()
        assert sT.dtype == sdt
        y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
        check_close("y", y, y_ref, torch.bfloat16)
        check_close("sT", sT, sT_ref, torch.bfloat16)


def test_chunk_split_consistency(op, oracle):
    # chunked prefill then continue from the returned fp32 state == one long call (to bf16 tolerance)
    B, T, H, N = 2, 256, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 52, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    op.algo = CHUNK
    s0 = ins[6].cuda()
    cut = 96
    a = [x[:, :cut].contiguous() for x in dev[:4]] + [dev[4]]
    b = [x[:, cut:].contiguous() for x in dev[:4]] + [dev[4]]
    ya, sa = op(*a, return_state=True, init_state=s0)
    yb, sb = op(*b, return_state=True, init_state=sa)
    y_ref, s_ref = oracle.forward_c(*ref, N, to_np(s0))
    check_close("y", torch.cat([ya, yb], 1), y_ref, torch.bfloat16)
    check_close("sT", sb, s_ref, torch.bfloat16)


def test_chunk_falls_back_on_extreme_decay(op, oracle):
    # a decay the tile scaling cannot represent: the affected (b, h) workgroups redo their pair with
    # the exact per-timestep code inside the same launch, the others keep their MFMA results
    B, T, H, N = 2, 128, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 53)
    ins[3][1, 40:60, 70:90] = 6.0     # exp(6) = 403 per step: far beyond the limit
    ins[3][0, 5, 3] = 20.0            # decay exactly 0
    ins[3][0, 90:100] = -1e9          # decay exactly 1
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.bfloat16)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.bfloat16)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], N)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.bfloat16, is_grad=True)


# fp16 tensors on the chunked kernels (training pair: y and gradients fp32, torch_rwkv_kernel.py:35):
# r, k, w are unpacked exactly from fp16, v and gy reach the MFMAs through bf16 copies.
@pytest.mark.parametrize("B,T,H", [(1, 32, 1), (2, 64, 2), (2, 100, 1), (1, 129, 3), (2, 1000, 2), (1, 2048, 1),
                                   (1, 16, 1), (1, 48, 1), (2, 333, 2), (3, 1024, 4), (1, 80, 5), (75, 64, 4), (300, 32, 1)])
def test_chunk_fwd_bwd_f16(op, oracle, B, T, H):
    _case(op, oracle, B, T, H, 140 + T, torch.float16, CHUNK, tol=torch.float16)


def test_chunk_f16_falls_back_on_extreme_decay(op, oracle):
    # as test_chunk_falls_back_on_extreme_decay: the exact second pass reads the fp16 v and the fp32 gy
    B, T, H, N = 2, 128, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 54)
    ins[3][1, 40:60, 70:90] = 6.0
    ins[3][0, 5, 3] = 20.0
    ins[3][0, 90:100] = -60000.0      # (fp16 range) decay exactly 1
    dev, ref = cast_inputs(ins[:5], torch.float16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.float32)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
    assert y.dtype == torch.float32
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.float16)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], N)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.float16, is_grad=True)


def test_f16_chunked_training_pair_is_opt_in(op, oracle):
    # AUTO keeps fp16 tensors at fp32 accuracy (the full-precision chunk form, fp32 chunk states saved for the
    # backward; the same y with and without a gradient); the bf16-operand pair runs on request only
    from rwkv_kernel import _native
    lib = _native.load()
    full = 2 * 2 * (256 // 32) * 64 * 64 * 4
    assert lib.wkv6_saved_bytes(_native.F16, _native.ALGO_AUTO, 2, 256, 128, 2) == full
    assert lib.wkv6_saved_bytes(_native.F32, _native.ALGO_AUTO, 2, 256, 128, 2) == full
    assert lib.wkv6_saved_bytes(_native.F16, _native.ALGO_SCAN, 2, 256, 128, 2) == 0
    assert lib.wkv6_saved_bytes(_native.F16, _native.ALGO_CHUNK, 2, 256, 128, 2) > full
    assert lib.wkv6_saved_bytes(_native.BF16, _native.ALGO_AUTO, 2, 256, 128, 2) > 0
    y_train, _ = _case(op, oracle, 2, 256, 2, 77, torch.float16, 0)          # fp32 tolerance (1e-4 / 1e-3)
    ins = oracle.make_inputs(2, 256, 2, 64, 77)
    dev, _ = cast_inputs(ins[:5], torch.float16)
    op.algo = 0
    with torch.no_grad():
        y_eval, _ = op(*dev)
    assert torch.equal(y_eval, y_train.detach())


# More (batch, head) pairs than the chip has compute units: a forward workgroup then runs several
# pairs back to back through one pipeline (the state, the head's u, the saved states and the
# fallback flag all switch at the pair boundaries).
@pytest.mark.parametrize("B,T,H", [(75, 64, 4), (43, 150, 7), (300, 32, 1), (1100, 16, 8)])   # the last: more than 32 pairs per compute unit
def test_chunk_many_pairs_fwd_bwd_bf16(op, oracle, B, T, H):
    _case(op, oracle, B, T, H, 90 + T, torch.bfloat16, CHUNK)


def test_chunk_many_pairs_state_in_out(op, oracle):
    B, T, H, N = 90, 130, 4, 64
    ins = oracle.make_inputs(B, T, H, N, 55, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    op.algo = CHUNK
    for sdt in (torch.bfloat16, torch.float32):
        s_dev, s_ref = cast_inputs([ins[6][:7]], sdt)
        smap = [(3 * i) % 7 for i in range(B)]
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
        torch.cuda.synchronize()
        y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
        check_close("y", y, y_ref, torch.bfloat16)
        check_close("sT", sT, sT_ref, torch.bfloat16)


def test_chunk_many_pairs_fall_back_pair_by_pair(op, oracle):
    # pairs 1 and 300 of 320 leave the representable range: each is redone exactly, whichever
    # position it has in its workgroup's list, and the others keep their MFMA results
    B, T, H, N = 80, 128, 4, 64
    ins = oracle.make_inputs(B, T, H, N, 56)
    ins[3][0, 40:60, 70:90] = 6.0        # pair (0, 1)
    ins[3][75, 100:120, 10:20] = 6.0     # pair (75, 0) = 300
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.bfloat16)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.bfloat16)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], N)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.bfloat16, is_grad=True)


# Fused output stage (inference): out = group_norm(y) * gate straight from the kernel, y never stored.
# Checked against the oracle's y (float64, fed the bf16-rounded inputs) pushed through the float64
# restatement of the model's group norm and gate.  Tolerance: the bf16 one of the operator,
# relative to the largest reference value (the kernel normalises the bf16-rounded y, as a caller
# would).
@pytest.mark.parametrize("B,T,H,with_state", [(2, 64, 2, False), (3, 150, 2, True), (1, 1000, 3, False),
                                              (70, 96, 4, True), (1, 16, 1, False), (5, 1, 3, True), (2, 1, 2, False),
                                              (1, 2600, 2, True), (2, 2048, 3, False)])   # the last two: in time segments
def test_fused_group_norm_gate(op, oracle, B, T, H, with_state):
    N = 64
    ins = oracle.make_inputs(B, T, H, N, 70 + T, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    g = torch.Generator().manual_seed(T)
    gate = torch.randn(B, T, H * N, generator=g)
    gate_dev, gate_ref = cast_inputs([gate], torch.bfloat16)
    scale = torch.rand(H, N, generator=g) + 0.5
    offset = torch.randn(H, N, generator=g) * 0.3
    s0 = ins[6].float() if with_state else None
    out, sT = op.forward_gn_gate(*dev, gate_dev[0], scale.cuda(), offset.cuda(), 64e-5, return_state=True,
                                 init_state=s0.cuda() if with_state else None)
    torch.cuda.synchronize()
    y_ref, sT_ref = oracle.forward_c(*ref, N, to_np(s0) if with_state else None)
    want = oracle.group_norm_gate_np(y_ref, gate_ref[0], scale.numpy(), offset.numpy(), N, 64e-5)
    check_close("out", out, want, torch.bfloat16)
    check_close("sT", sT, sT_ref, torch.bfloat16)


def _fused_training_case(op, oracle, B, T, H, seed, wild=False):
    """The differentiable fused call against float64: the oracle's y, torch's layer_norm autograd for
    the norm and the gate (its gradient wrt y rounded to bf16, as the kernel hands it on), the oracle's
    backward for the operator."""
    N = 64
    C = H * N
    ins = oracle.make_inputs(B, T, H, N, seed)
    if wild:
        ins[3][0, 8:24, 5:40] = 6.0      # one pair redoes itself with the exact per-timestep code
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 1)
    gate_dev, gate_ref = cast_inputs([torch.randn(B, T, C, generator=g)], torch.bfloat16)
    # the gradient arriving is zero where the norm is ill-conditioned (see flat_heads): what is compared is
    # the kernels' arithmetic, not the norm's magnification of y's rounding; `out` is compared everywhere
    from _util import check_composite, flat_heads, fused_stage_reference
    y_ref, _ = oracle.forward_c(*ref, N)
    keep = torch.tensor(~flat_heads(y_ref, N)).view(B, T, H, 1).expand(B, T, H, N).reshape(B, T, C)
    gout_dev, gout_ref = cast_inputs([torch.randn(B, T, C, generator=g) * keep], torch.bfloat16)
    scale = (torch.rand(H, N, generator=g) + 0.5).cuda().requires_grad_(True)
    offset = (torch.randn(H, N, generator=g) * 0.3).cuda().requires_grad_(True)
    leaves = [x.clone().requires_grad_(True) for x in dev] + [gate_dev[0].clone().requires_grad_(True)]
    op.algo = CHUNK
    out, none = op.forward_gn_gate(*leaves, scale, offset, 64e-5)
    assert none is None and out.dtype == torch.bfloat16
    out.backward(gout_dev[0])
    torch.cuda.synchronize()
    # float64 reference; tolerance: see check_composite (the operator alone is held to 1e-2 by the tests
    # above, the norm's backward by test_group_norm_gate_backward_kernel)
    want = fused_stage_reference(oracle, ref, gate_ref[0], gout_ref[0], to_np(scale), to_np(offset), N, 64e-5, y_ref)
    check_composite("out", out, want["out"])
    check_composite("ggate", leaves[5].grad, want["ggate"])
    check_composite("gscale", scale.grad, want["gscale"])
    check_composite("goffset", offset.grad, want["goffset"])
    for name, leaf in zip("gr gk gv gw gu".split(), leaves[:5]):
        check_composite(name, leaf.grad, want[name])


@pytest.mark.parametrize("B,T,H", [(2, 37, 3), (4, 256, 8)])
def test_group_norm_gate_backward_kernel(op, B, T, H):
    """wkv6_gn_gate_backward alone, through the C ABI, against torch's layer_norm autograd in float64 on
    the same (bf16-rounded) y, gate, gout and the statistics of that y."""
    from rwkv_kernel import _native
    lib = _native.load()
    N = 64
    C = H * N
    g = torch.Generator().manual_seed(B * T + H)
    y, gate, gout = (torch.randn(B, T, C, generator=g).mul(s).to(torch.bfloat16).cuda() for s in (3.0, 1.0, 1.0))
    scale = (torch.rand(H, N, generator=g) + 0.5).cuda()
    offset = (torch.randn(H, N, generator=g) * 0.3).cuda()
    eps = 64e-5
    yt = y.double().cpu().requires_grad_(True)
    gt = gate.double().cpu().requires_grad_(True)
    st = scale.double().cpu().requires_grad_(True)
    ot = offset.double().cpu().requires_grad_(True)
    x = yt.view(B, T, H, N)
    mean = x.mean(-1)
    rstd = 1.0 / torch.sqrt(x.var(-1, unbiased=False) + eps)
    stats = torch.stack([mean, rstd], -1).detach().float().cuda().contiguous()
    out = (torch.nn.functional.layer_norm(x, (N,), eps=eps) * st + ot).view(B, T, C) * gt
    out.backward(gout.double().cpu())
    gy, gg = torch.empty_like(y), torch.empty_like(y)
    gs = torch.full((C,), 7.0, device="cuda")       # (the call zeroes the sums itself)
    go = torch.full((C,), 7.0, device="cuda")
    st_ = torch.cuda.current_stream().cuda_stream
    _native.check(lib.wkv6_gn_gate_backward(st_, _native.BF16, B, T, C, H, gout.data_ptr(), y.data_ptr(), stats.data_ptr(), gate.data_ptr(),
                                            scale.data_ptr(), offset.data_ptr(), gy.data_ptr(), gg.data_ptr(), gs.data_ptr(), go.data_ptr()))
    torch.cuda.synchronize()
    check_close("gy", gy, yt.grad.numpy(), torch.bfloat16, is_grad=True)
    check_close("ggate", gg, gt.grad.numpy(), torch.bfloat16, is_grad=True)
    check_close("gscale", gs.cpu().double().numpy().reshape(H, N), st.grad.numpy(), torch.float32, is_grad=True)
    check_close("goffset", go.cpu().double().numpy().reshape(H, N), ot.grad.numpy(), torch.float32, is_grad=True)


# (the last shape: one layer of the training benchmark, B = 8, T = 1024, 32 heads)
@pytest.mark.parametrize("B,T,H", [(2, 64, 2), (3, 150, 2), (1, 1000, 3), (8, 256, 8), (75, 64, 4), (8, 1024, 32)])
def test_fused_group_norm_gate_training(op, oracle, B, T, H):
    _fused_training_case(op, oracle, B, T, H, 300 + T)


def test_fused_group_norm_gate_training_twice_over_one_graph(op, oracle):
    """backward(retain_graph=True) and a second backward over the same graph: the first consumes the saved
    block, the second rebuilds the states; both return the same gradients (those of the operator to the
    bf16 tolerance, the gate's bit for bit, the norm's two sums to fp32 rounding)."""
    B, T, H, N = 3, 128, 2, 64
    C = H * N
    ins = oracle.make_inputs(B, T, H, N, 909)
    dev, _ = cast_inputs(ins[:5], torch.bfloat16)
    g = torch.Generator().manual_seed(910)
    gate = torch.randn(B, T, C, generator=g).to(torch.bfloat16).cuda().requires_grad_(True)
    gout = torch.randn(B, T, C, generator=g).to(torch.bfloat16).cuda()
    scale = (torch.rand(H, N, generator=g) + 0.5).cuda().requires_grad_(True)
    offset = (torch.randn(H, N, generator=g) * 0.3).cuda().requires_grad_(True)
    leaves = [x.clone().requires_grad_(True) for x in dev] + [gate, scale, offset]
    op.algo = CHUNK
    out, _ = op.forward_gn_gate(*leaves, 64e-5)
    first = torch.autograd.grad(out, leaves, gout, retain_graph=True)
    second = torch.autograd.grad(out, leaves, gout)
    torch.cuda.synchronize()
    for name, a, b in zip("gr gk gv gw gu ggate gscale goffset".split(), first, second):
        if name == "ggate":
            assert torch.equal(a, b), name
        elif name in ("gscale", "goffset"):          # (atomic sums: the order of the additions varies)
            check_close(name + " (second backward)", b, to_np(a), torch.float32, is_grad=True)
        else:
            check_close(name + " (second backward)", b, to_np(a), torch.bfloat16, is_grad=True)


def test_fused_group_norm_gate_training_on_a_fallback_pair(op, oracle):
    _fused_training_case(op, oracle, 2, 128, 2, 333, wild=True)


@pytest.mark.parametrize("B,T,H,wild", [(1, 2048, 2, False), (2, 1024, 3, False), (1, 2048, 32, False), (1, 4096, 4, True)])
def test_fused_group_norm_gate_training_in_time_segments(op, oracle, B, T, H, wild):
    # few pairs and a long sequence: the operator's training pair runs in time segments, and the output stage
    # is part of their second pass (tile form; with 32 heads the segments fill the chip and run on the block
    # form; the last case has pairs that fall back to the per-timestep pass inside their segment)
    from rwkv_kernel import _native
    lib = _native.load()
    assert lib.wkv6_forward_gn_gate_save_supported(_native.BF16, B, T, H * 64, H) == 1
    _fused_training_case(op, oracle, B, T, H, 340 + H, wild=wild)


def test_fused_group_norm_gate_on_a_fallback_pair(op, oracle):
    # a pair that leaves the chunked form's range is redone exactly and then normalised in place
    B, T, H, N = 2, 128, 2, 64
    ins = oracle.make_inputs(B, T, H, N, 77)
    ins[3][1, 40:60, 70:90] = 6.0
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    g = torch.Generator().manual_seed(5)
    gate_dev, gate_ref = cast_inputs([torch.randn(B, T, H * N, generator=g)], torch.bfloat16)
    scale, offset = torch.rand(H, N, generator=g) + 0.5, torch.randn(H, N, generator=g) * 0.3
    out, _ = op.forward_gn_gate(*dev, gate_dev[0], scale.cuda(), offset.cuda())
    torch.cuda.synchronize()
    want = oracle.group_norm_gate_np(oracle.forward_c(*ref, N)[0], gate_ref[0], scale.numpy(), offset.numpy(), N)
    check_close("out", out, want, torch.bfloat16)


# Gradients through the state (an extension of the reference's stateful call): loss =
# sum(y*gy) + sum(S_T*gS) with S_0 given; checked against the float64 adjoint-form oracle (itself
# pinned by torch.autograd through the python loop).
def _state_grad_case(op, oracle, B, T, H, seed, dtype, algo, with_s0=True, with_gs=True, wild=False):
    N = 64
    ins = oracle.make_inputs(B, T, H, N, seed, with_state=True)
    if wild:
        ins[3][B - 1, T // 3:T // 3 + 20, 5:25] = 6.0
    odt = out_dtype(dtype)
    dev, ref = cast_inputs(ins[:5], dtype)
    gy_dev, gy_ref = cast_inputs(ins[5:6], odt)
    s0 = ins[6].float() * 3 if with_s0 else None
    gS = torch.randn(B, H, N, N, generator=torch.Generator().manual_seed(seed)) if with_gs else None
    leaves = [x.clone().requires_grad_(True) for x in dev]
    s0_dev = s0.cuda().requires_grad_(True) if with_s0 else None
    op.algo = algo
    y, sT = op(*leaves, return_state=True, init_state=s0_dev)
    assert sT.dtype == torch.float32 and y.requires_grad
    loss = (y.float() * gy_dev[0].float()).sum()
    if with_gs:
        loss = loss + (sT * gS.cuda()).sum()
    got = torch.autograd.grad(loss, leaves + ([s0_dev] if with_s0 else []))
    torch.cuda.synchronize()
    want = oracle.backward_state_c(*ref, gy_ref[0], N, None if s0 is None else to_np(s0), None if gS is None else to_np(gS))
    y_ref, sT_ref = oracle.forward_c(*ref, N, None if s0 is None else to_np(s0))
    check_close("y", y.detach(), y_ref, odt)
    check_close("sT", sT.detach(), sT_ref, odt)
    names = "gr gk gv gw gu".split() + (["gs0"] if with_s0 else [])
    for name, g, gr in zip(names, got, want):
        check_close(name, to_np(g).reshape(gr.shape), gr, odt, is_grad=True)
    if not with_s0:
        assert float(got[3][:, 0].abs().max()) == 0.0      # zero initial state: the first decay reaches nothing
    if not with_gs:
        assert float(got[3][:, -1].abs().max()) == 0.0


@pytest.mark.parametrize("dt,T", [("f32", 37), ("f32", 1), ("bf16", 50), ("f16", 16)])
def test_state_gradients_scan(op, oracle, dt, T):
    _state_grad_case(op, oracle, 2, T, 2, 80 + T, DTYPES[dt], SCAN)


@pytest.mark.parametrize("B,T,H", [(2, 64, 2), (2, 150, 1), (1, 512, 3)])
def test_state_gradients_chunk_bf16(op, oracle, B, T, H):
    _state_grad_case(op, oracle, B, T, H, 85 + T, torch.bfloat16, CHUNK)


def test_state_gradients_one_sided(op, oracle):
    _state_grad_case(op, oracle, 2, 96, 2, 91, torch.bfloat16, CHUNK, with_s0=False, with_gs=True)
    _state_grad_case(op, oracle, 2, 96, 2, 92, torch.bfloat16, CHUNK, with_s0=True, with_gs=False)
    _state_grad_case(op, oracle, 2, 40, 2, 93, torch.float32, SCAN, with_s0=False, with_gs=True)
    _state_grad_case(op, oracle, 2, 40, 2, 94, torch.float32, SCAN, with_s0=True, with_gs=False)


@pytest.mark.parametrize("with_s0,with_gs", [(True, True), (False, True), (True, False), (False, False)])
def test_state_gradients_in_time_segments(op, oracle, with_s0, with_gs):
    # few pairs, long sequence: wkv6_backward_with_state rebuilds the segments' states, chains the
    # reverse state from the arriving gradient and returns what leaves the first segment as dL/dS_0
    _state_grad_case(op, oracle, 1, 2048, 3, 98, torch.bfloat16, CHUNK, with_s0=with_s0, with_gs=with_gs)


def test_state_gradients_in_time_segments_with_a_fallback_segment(op, oracle):
    _state_grad_case(op, oracle, 2, 2048, 1, 99, torch.bfloat16, CHUNK, wild=True)


def test_state_gradients_on_a_fallback_pair(op, oracle):
    _state_grad_case(op, oracle, 2, 128, 2, 95, torch.bfloat16, CHUNK, wild=True)


def test_backpropagation_over_two_pieces_equals_one_piece(op):
    # the property the state gradient exists for: a sequence cut in two, the state and its gradient
    # handed across the cut, gives the gradients of the uncut sequence (fp32, exact kernels)
    from oracle import wkv6_ref
    B, T, H, N, cut = 2, 96, 2, 64, 40
    ins = wkv6_ref.make_inputs(B, T, H, N, 96)
    r, k, v, w, u, gy = (x.float().cuda() for x in ins[:6])
    op.algo = SCAN
    whole = [x.clone().requires_grad_(True) for x in (r, k, v, w, u)]
    y, _ = op(*whole)
    g_whole = torch.autograd.grad((y * gy).sum(), whole)
    parts = [x.clone().requires_grad_(True) for x in (r, k, v, w, u)]
    a = [x[:, :cut].contiguous() for x in parts[:4]] + [parts[4]]
    b = [x[:, cut:].contiguous() for x in parts[:4]] + [parts[4]]
    ya, sa = op(*a, return_state=True)
    yb, _ = op(*b, return_state=True, init_state=sa)
    g_parts = torch.autograd.grad((torch.cat([ya, yb], 1) * gy).sum(), parts)
    for name, x, z in zip("gr gk gv gw gu".split(), g_parts, g_whole):
        err = float((x - z).abs().max()) / max(1e-12, float(z.abs().max()))
        assert err <= 2e-5, (name, err)


# Few pairs, long sequence: with the optional forward workspace the sequence runs as time segments
# side by side (two passes joined by the affine state map of a segment).
@pytest.mark.parametrize("B,T,H,sdt", [(1, 2048, 2, torch.float32), (2, 2304, 1, torch.bfloat16), (3, 4096, 5, torch.float32), (12, 2048, 4, torch.float32),
                                       (1, 5000, 2, torch.float32), (1, 3000, 3, torch.bfloat16), (1, 4097, 2, torch.float32)])   # single sequences that leave a remainder (the last: of one token)
def test_forward_in_time_segments(op, oracle, B, T, H, sdt):
    from rwkv_kernel import _native
    N = 64
    lib = _native.load()
    assert lib.wkv6_forward_workspace_bytes(_native.BF16, CHUNK, B, T, H * N, H) > 0
    assert lib.wkv6_forward_workspace_bytes(_native.BF16, CHUNK, 8, 1024, 2048, 32) == 0    # fills the chip as it is
    # no equal segments: only a single sequence can leave a remainder behind them
    assert (lib.wkv6_forward_workspace_bytes(_native.BF16, CHUNK, B, T + 64, H * N, H) > 0) == (B == 1)
    ins = oracle.make_inputs(B, T, H, N, 60 + B, with_state=True)
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    kinds = min(2, B)
    s_dev, s_ref = cast_inputs([ins[6][:kinds]], sdt)
    smap = [(b + 1) % kinds for b in range(B)]
    op.algo = CHUNK
    y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
    torch.cuda.synchronize()
    y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
    check_close("y", y, y_ref, torch.bfloat16)
    check_close("sT", sT, sT_ref, torch.bfloat16)
    # a segment that leaves the chunked form's range is redone exactly in both passes
    ins[3][0, T // 2 + 30:T // 2 + 50, 20:40] = 6.0
    dev2, ref2 = cast_inputs(ins[:5], torch.bfloat16)
    y2, sT2 = op(*dev2, return_state=True, init_state=s_dev[0], state_map=smap)
    y2_ref, sT2_ref = oracle.forward_c(*ref2, N, s_ref[0], smap)
    check_close("y with an exact segment", y2, y2_ref, torch.bfloat16)
    check_close("sT with an exact segment", sT2, sT2_ref, torch.bfloat16)
    # and from a zero state, with and without a final state
    y0, s0T = op(*dev, return_state=True)
    y1, _ = op(*dev)
    torch.cuda.synchronize()
    check_close("y vs one pass", y0, to_np(y1).astype(np.float64), torch.bfloat16)
    check_close("sT zero", s0T, oracle.forward_c(*ref, N)[1], torch.bfloat16)


@pytest.mark.parametrize("B,T,H,P", [(1, 2048, 2, 8), (2, 4096, 1, 16), (3, 3072, 5, 8), (1, 8192, 20, 8), (13, 2048, 5, 2),
                                     (2, 1024, 3, 4), (1, 1536, 2, 4)])
def test_training_pair_in_time_segments(op, oracle, B, T, H, P):
    """Few pairs, long sequence: forward_save + backward_saved_sum run the sequence as P segments side
    by side (joined by the affine state map and, for the reverse state, its transpose); against the
    oracle over the whole sequence."""
    from rwkv_kernel import _native

    lib = _native.load()
    C = H * 64
    whole = B * H * (T // 64) * 64 * 64 * 4   # chunk states of the sequences in one piece
    assert lib.wkv6_saved_bytes(_native.BF16, CHUNK, B, T, C, H) >= whole + B * P * H * 2 * 64 * 64 * 4   # segment states
    _, grads = _case(op, oracle, B, T, H, 90 + H, torch.bfloat16, CHUNK)
    gw = grads[3]
    assert float(gw[:, 0].abs().max()) == 0.0 and float(gw[:, -1].abs().max()) == 0.0


def test_training_pair_in_time_segments_with_fallback_segments(op, oracle):
    # segments whose decay the tile scaling cannot represent are redone by the exact per-timestep
    # code in every pass (forward passes, both backward passes); decay exactly 0 and exactly 1
    # across segment boundaries
    B, T, H, N = 1, 2048, 3, 64          # 8 segments of 256 tokens
    ins = oracle.make_inputs(B, T, H, N, 97)
    ins[3][0, 700:720, 70:90] = 6.0      # inside segment 2, head 1
    ins[3][0, 1279:1282, 130:140] = 20.0  # decay 0 around the boundary of segments 4 and 5, head 2
    ins[3][0, 250:260] = -1e9            # decay 1 across the boundary of segments 0 and 1
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.bfloat16)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.bfloat16)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], N)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.bfloat16, is_grad=True)


def test_chunk_matches_scan_on_padding_mask(op, oracle):
    B, T, H, N = 1, 96, 1, 64
    ins = oracle.make_inputs(B, T, H, N, 54)
    ins[3][:, 20:50] = -1e9
    ins[1][:, 20:50] = 0
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    op.algo = CHUNK
    y, _ = op(*dev)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.bfloat16)


@pytest.mark.parametrize("B,T,H", [(40, 128, 8), (5, 100, 64), (100, 64, 3), (300, 37, 1), (33, 200, 10), (130, 512, 2)])
def test_chunk_backward_with_more_pairs_than_compute_units(op, oracle, B, T, H):
    """More (batch, head) pairs than the GPU has compute units and a short sequence: the backward runs one
    workgroup per compute unit, each taking several pairs back to back (different batch rows of one
    head); every pair's gradients, and gu summed over the batch, against the oracle.  Head counts
    that divide the number of compute units and ones that do not, one chunk per pair and several, a
    ragged last chunk."""
    _case(op, oracle, B, T, H, 500 + T, torch.bfloat16, CHUNK)


@pytest.mark.parametrize("B,T,H", [(208, 51, 7), (323, 134, 3), (60, 33, 12), (146, 69, 12), (140, 290, 3), (49, 273, 6),
                                   (29, 475, 9), (49, 173, 7), (109, 53, 3), (99, 167, 5)])
def test_chunk_many_pairs_drawn_shapes(op, oracle, B, T, H):
    # shapes drawn once at random among those with more pairs than compute units: ragged lengths, head
    # counts that do not divide the number of compute units, workgroups with unequal numbers of pairs
    _case(op, oracle, B, T, H, 700 + B, torch.bfloat16, CHUNK)


def test_chunk_backward_with_more_pairs_than_a_workgroup_keeps_flags_for(op, oracle):
    """16 500 single-head sequences of 32 tokens: more than 64 pairs per compute unit, so the grid of the
    several-pairs backward is a multiple of its usual size.  The rows are independent: a few of them
    (first, last, around the places where a workgroup's pair list wraps) against the oracle, and gu
    summed over all rows against its closed form  sum_{b,t} r k <v, gy>  in float64."""
    B, T, H, N = 16500, 32, 1, 64
    g = torch.Generator().manual_seed(91)
    mk = lambda: torch.randn(B, T, N, generator=g).to(torch.bfloat16)
    r, k, v, gy = mk(), mk(), mk(), mk()
    w = (torch.rand(B, T, N, generator=g) * 7 - 6).to(torch.bfloat16)
    u = (torch.randn(H, N, generator=g) * 0.5).to(torch.bfloat16)
    dev = [x.cuda() for x in (r, k, v, w, u, gy)]
    y, grads = _run_fwd_bwd(op, dev, CHUNK)
    rows = [0, 1, 255, 256, 257, 511, 512, 8191, 8192, 16383, 16384, 16385, B - 2, B - 1]
    sub = [to_np(x[rows]) for x in (r, k, v, w)] + [to_np(u)]
    check_close("y", y[rows], oracle.forward_c(*sub, N)[0], torch.bfloat16)
    g_ref = oracle.backward_c(*sub, to_np(gy[rows]), N)
    for name, got, want in zip("gr gk gv gw".split(), grads[:4], g_ref[:4]):
        check_close(name, got[rows], want, torch.bfloat16, is_grad=True)
    rd, kd, vd, gd = (x.cuda().double() for x in (r, k, v, gy))
    gu_ref = (rd * kd * (vd * gd).sum(-1, keepdim=True)).sum((0, 1)).cpu().numpy().reshape(H, N)
    check_close("gu", to_np(grads[4]).reshape(H, N), gu_ref, torch.bfloat16, is_grad=True)


def test_chunk_many_pairs_fall_back_on_extreme_decay(op, oracle):
    # as test_chunk_falls_back_on_extreme_decay with 280 pairs: pairs that are a workgroup's first and
    # ones that are its second leave the chunked form's range and are redone exactly after the
    # workgroup's last pair, their neighbours in the same workgroup keep their MFMA results
    B, T, H, N = 70, 128, 4, 64
    ins = oracle.make_inputs(B, T, H, N, 57)
    ins[3][0, 40:60, 70:90] = 6.0          # pair (0, 1)
    ins[3][69, 10:30, 200:230] = 6.0       # pair (69, 3): index 279, the second pair of its workgroup
    ins[3][66, 100:110, 0:64] = 7.0        # pair (66, 0): index 264
    ins[3][3, 90:100] = -1e9               # decay exactly 1
    dev, ref = cast_inputs(ins[:5], torch.bfloat16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], torch.bfloat16)
    y, grads = _run_fwd_bwd(op, dev + gy_dev, CHUNK)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.bfloat16)
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref[0], N)):
        check_close(name, to_np(g).reshape(gr.shape), gr, torch.bfloat16, is_grad=True)


@pytest.mark.parametrize("B,T,H", [(2, 320, 2), (150, 192, 2)])
def test_plain_backward_equals_saved_backward(op, oracle, B, T, H):
    # wkv6_backward (recomputes the chunk states) and wkv6_backward_saved (takes them from the
    # forward) agree to rounding (the two sweeps scale k differently before the bf16 rounding),
    # and both meet the tolerance against the oracle; with few pairs and with more pairs than compute units
    from rwkv_kernel import _native

    lib = _native.load()
    N = 64
    C = H * N
    ins = oracle.make_inputs(B, T, H, N, 77)
    dev, _ = cast_inputs(ins[:6], torch.bfloat16)
    r, k, v, w, u, gy = dev
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    res = []
    for mode in ("plain", "saved"):
        y = torch.empty_like(r)
        outs = [torch.empty_like(r) for _ in range(4)] + [torch.empty(B, C, dtype=r.dtype, device="cuda")]
        n = lib.wkv6_saved_bytes(_native.BF16, CHUNK, B, T, C, H)
        assert n >= lib.wkv6_backward_workspace_bytes_ex(_native.BF16, CHUNK, B, T, C, H) > 0   # + arrival counters
        buf = torch.empty(n, dtype=torch.uint8, device="cuda")
        if mode == "plain":
            _native.check(lib.wkv6_forward_ex(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), None, 0))
            _native.check(lib.wkv6_backward_ex(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                               *[P(o) for o in outs], P(buf), n))
        else:
            _native.check(lib.wkv6_forward_save(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), P(buf), n))
            _native.check(lib.wkv6_backward_saved(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                  *[P(o) for o in outs], P(buf), n))
        torch.cuda.synchronize()
        res.append([y] + outs)
    assert torch.equal(res[0][0], res[1][0])
    _, ref = cast_inputs(ins[:6], torch.bfloat16)
    g_ref = oracle.backward_c(*ref[:5], ref[5], N)
    for which in res:
        for name, g, gr in zip("gr gk gv gw".split(), which[1:5], g_ref):
            check_close(name, g, gr, torch.bfloat16, is_grad=True)
        check_close("gu", to_np(which[5]).sum(0).reshape(H, N), g_ref[4], torch.bfloat16, is_grad=True)
    for a, b in zip(res[0][1:5], res[1][1:5]):
        assert (a.float() - b.float()).abs().max() <= 5e-3 * b.float().abs().max()
    assert lib.wkv6_saved_bytes(_native.F32, SCAN, B, T, C, H) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("B,T,H,dt", [(8, 256, 8, "bf16"), (5, 100, 3, "bf16"), (1, 64, 2, "bf16"), (3, 40, 2, "f32")])
def test_fused_gu_batch_sum(op, oracle, B, T, H, dt):
    """wkv6_backward_saved_sum: gu_sum is the sum over the batch of the partials it also returns
    (summed in fp32, rounded once: what torch.sum does for the caller, rwkv_kernel/torch_rwkv_kernel.py:73),
    on two consecutive backward calls over the same hand-over buffer, and for head counts that do
    and do not divide over the XCDs evenly."""
    from rwkv_kernel import _native
    lib = _native.load()
    N, C = 64, H * 64
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[dt]
    code = {"bf16": _native.BF16, "f32": _native.F32}[dt]
    r, k, v, w, u, gy = (x.to(dtype).cuda().contiguous() for x in oracle.make_inputs(B, T, H, N, 11))
    y = torch.empty_like(r)
    gr, gk, gv, gw = (torch.empty_like(r) for _ in range(4))
    # (for the per-timestep path nothing is saved and the same buffer is just the backward's workspace)
    n = max(lib.wkv6_saved_bytes(code, _native.ALGO_AUTO, B, T, C, H),
            lib.wkv6_backward_workspace_bytes_ex(code, _native.ALGO_AUTO, B, T, C, H), 16)
    saved = torch.empty(n, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    _native.check(lib.wkv6_forward_save(st, code, _native.ALGO_AUTO, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), P(saved), n))
    for _ in range(2):
        gu = torch.full((B, C), float("nan"), dtype=dtype, device="cuda")
        gs = torch.full((C,), float("nan"), dtype=dtype, device="cuda")
        _native.check(lib.wkv6_backward_saved_sum(st, code, _native.ALGO_AUTO, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                  P(gr), P(gk), P(gv), P(gw), P(gu), P(gs), P(saved), n))
        torch.cuda.synchronize()
        want = torch.sum(gu.float(), 0).to(dtype)
        assert torch.isfinite(gs).all()
        assert torch.equal(gs, want) or float((gs.float() - want.float()).abs().max()) <= 2 ** -7 * float(want.float().abs().max())
    # and the partials are the ones the plain call gives
    gu2 = torch.empty_like(gu)
    _native.check(lib.wkv6_backward_saved(st, code, _native.ALGO_AUTO, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                          P(gr), P(gk), P(gv), P(gw), P(gu2), P(saved), n))
    torch.cuda.synchronize()
    assert torch.equal(gu, gu2)


@pytest.mark.gpu
@pytest.mark.parametrize("B,T,H", [(2, 256, 4), (1, 2048, 3), (70, 128, 4)])   # the second: seven launches (time segments); the third: several pairs per workgroup
def test_training_pair_replays_in_a_hip_graph(op, oracle, B, T, H):
    """forward_save + backward_saved_sum captured once into a graph (the library allocates nothing
    and only enqueues on the given stream), replayed several times with eager work and
    synchronisations in between; every replay must reproduce the eager results bit for bit."""
    from rwkv_kernel import _native
    lib = _native.load()
    N = 64
    C = H * N
    r, k, v, w, u, gy = (x.to(torch.bfloat16).cuda().contiguous() for x in oracle.make_inputs(B, T, H, N, 21))
    n = lib.wkv6_saved_bytes(_native.BF16, _native.ALGO_AUTO, B, T, C, H)
    saved = torch.empty(n, dtype=torch.uint8, device="cuda")
    outs = {name: torch.empty_like(r) for name in ("y", "gr", "gk", "gv", "gw")}
    outs["gu"] = torch.empty(B, C, dtype=r.dtype, device="cuda")
    outs["gs"] = torch.empty(C, dtype=r.dtype, device="cuda")
    P = lambda t: t.data_ptr()

    def step():
        st = torch.cuda.current_stream().cuda_stream
        _native.check(lib.wkv6_forward_save(st, _native.BF16, _native.ALGO_AUTO, B, T, C, H,
                                            P(r), P(k), P(v), P(w), P(u), P(outs["y"]), P(saved), n))
        _native.check(lib.wkv6_backward_saved_sum(st, _native.BF16, _native.ALGO_AUTO, B, T, C, H,
                                                  P(r), P(k), P(v), P(w), P(u), P(gy), P(outs["gr"]), P(outs["gk"]),
                                                  P(outs["gv"]), P(outs["gw"]), P(outs["gu"]), P(outs["gs"]), P(saved), n))

    step()
    torch.cuda.synchronize()
    eager = {name: t.clone() for name, t in outs.items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                      # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in outs.values():
            t.fill_(float("nan"))   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, t in outs.items():
            assert torch.equal(t, eager[name]), (rep, name)
