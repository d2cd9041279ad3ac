"""GPU parity tests of the full-precision chunk form (fp32 and fp16 tensors on the fp32 matrix instructions,
what WKV6_ALGO_AUTO runs for them from T = 64 on): called through the operator class and the C ABI, against
the float64 CPU oracle on the same seeded (and identically rounded) inputs, at the fp32 tolerances:
max|y - y_ref| <= 1e-4 (scaled by max|y_ref| / 64 above 64), gradients max|g - g_ref| / max|g_ref| <= 1e-3."""
import numpy as np
import pytest
import torch

from _util import cast_inputs, check_close, to_np

pytestmark = pytest.mark.gpu

AUTO, SCAN, CHUNK = 0, 1, 2
N = 64
DTYPES = {"f32": torch.float32, "f16": torch.float16}


@pytest.fixture(scope="module")
def op():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import rwkv_kernel

    return rwkv_kernel.RWKVKernelOperator(64, 1 << 16)


@pytest.fixture(scope="module")
def lib():
    from rwkv_kernel import _native

    return _native.load()


def _fwd_bwd(op, dev, gy, algo):
    op.algo = algo
    leaves = [x.clone().requires_grad_(True) for x in dev]
    y, none = op(*leaves)
    assert none is None
    y.backward(gy)
    torch.cuda.synchronize()
    return y, [x.grad for x in leaves]


def _check_grads(grads, g_ref, dtype, what=""):
    # fp16 gradients come back rounded to fp16 by the operator class: held to the 16-bit bound then
    tol = torch.float32 if dtype == torch.float32 else torch.float16
    for name, g, gr in zip("gr gk gv gw gu".split(), grads, g_ref):
        check_close(what + name, to_np(g).reshape(gr.shape), gr, tol, is_grad=True)


def _case(op, oracle, B, T, H, seed, dtype, edit=None, strict=False):
    print("case B=%d T=%d H=%d seed=%d dtype=%s" % (B, T, H, seed, dtype), flush=True)
    ins = oracle.make_inputs(B, T, H, N, seed)
    if edit:
        edit(ins)
    dev, ref = cast_inputs(ins[:5], dtype)
    gyd, gyr = cast_inputs(ins[5:6], torch.float32)
    y, grads = _fwd_bwd(op, dev, gyd[0], AUTO)
    assert y.dtype == torch.float32 and all(g.dtype == dtype for g in grads)
    y_ref, _ = oracle.forward_c(*ref, N)
    if strict:
        assert np.abs(to_np(y) - y_ref).max() <= 1e-4
    check_close("y", y, y_ref, torch.float32)
    _check_grads(grads, oracle.backward_c(*ref, gyr[0], N), dtype)
    return y, grads


def test_selected_from_64_tokens_on(lib):
    from rwkv_kernel import _native

    per_pair_chunk = 64 * 64 * 4
    for dt in (_native.F32, _native.F16):
        assert lib.wkv6_saved_bytes(dt, _native.ALGO_AUTO, 2, 64, 128, 2) == 2 * 2 * 2 * per_pair_chunk
        assert lib.wkv6_saved_bytes(dt, _native.ALGO_AUTO, 2, 100, 128, 2) == 2 * 2 * 4 * per_pair_chunk   # the last chunk is short
        assert lib.wkv6_saved_bytes(dt, _native.ALGO_AUTO, 2, 63, 128, 2) == 0      # short sequences: per-timestep kernels
        assert lib.wkv6_saved_bytes(dt, _native.ALGO_SCAN, 2, 256, 128, 2) == 0
    assert lib.wkv6_saved_bytes(_native.F32, _native.ALGO_CHUNK, 2, 256, 128, 2) == 2 * 2 * 8 * per_pair_chunk
    # the workspace of a backward without saved states holds the same chunk states (or the per-timestep pass's rows)
    assert lib.wkv6_backward_workspace_bytes_ex(_native.F32, _native.ALGO_AUTO, 2, 256, 128, 2) == 2 * 2 * 8 * per_pair_chunk
    assert lib.wkv6_backward_workspace_bytes_ex(_native.F32, _native.ALGO_SCAN, 2, 256, 128, 2) == 2 * 256 * 128 * 4


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_config1_forward_backward_fp32_strict(op, oracle, seed):
    # the fp32 correctness shape: B=2 T=128 H=4 N=64; max-abs(y) <= 1e-4
    _case(op, oracle, 2, 128, 4, seed, torch.float32, strict=True)


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("B,T,H", [(1, 64, 1), (2, 65, 2), (2, 95, 3), (2, 100, 2), (1, 333, 3), (3, 1024, 2), (1, 2080, 1)])
def test_shapes_and_ragged_ends(op, oracle, dt, B, T, H):
    _case(op, oracle, B, T, H, 100 + T, DTYPES[dt])


def test_more_pairs_than_compute_units(op, oracle):
    _case(op, oracle, 40, 96, 8, 7, torch.float32)


@pytest.mark.parametrize("dt", ["f32", "f16"])
def test_state_in_and_out(op, oracle, dt):
    B, T, H = 5, 170, 3
    ins = oracle.make_inputs(B, T, H, N, 21, with_state=True)
    dev, ref = cast_inputs(ins[:5], DTYPES[dt])
    s_dev, s_ref = cast_inputs([ins[6][:3]], torch.float32)
    smap = [2, 0, 1, 1, 2]
    op.algo = AUTO
    with torch.no_grad():
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
        y0, sT0 = op(*dev, return_state=True)
    torch.cuda.synchronize()
    y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
    check_close("y", y, y_ref, torch.float32)
    check_close("sT", sT, sT_ref, torch.float32, is_grad=True)
    y_ref0, sT_ref0 = oracle.forward_c(*ref, N)
    check_close("y from zero", y0, y_ref0, torch.float32)
    check_close("sT from zero", sT0, sT_ref0, torch.float32, is_grad=True)


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("B,T,H,with_s0,with_gs,wild", [(2, 64, 2, True, True, False), (2, 150, 1, True, True, False), (1, 512, 3, True, True, False),
                                                     (2, 96, 2, False, True, False), (2, 97, 2, True, False, False), (3, 128, 2, False, False, False),
                                                     (2, 160, 2, True, True, True), (260, 64, 1, True, True, False)])
def test_gradients_through_the_state(op, oracle, dt, B, T, H, with_s0, with_gs, wild):
    # loss = sum(y * gy) + sum(S_T * gS) with S_0 given: wkv6_backward_with_state on the full-precision chunk form (a
    # states-only forward from S_0, the backward with the reverse state started from gS), against the float64
    # adjoint-form oracle; one-sided cases, a pair redone per timestep, more pairs than compute units
    dtype = DTYPES[dt]
    print("state gradients B=%d T=%d H=%d %s s0=%d gS=%d wild=%d" % (B, T, H, dt, with_s0, with_gs, wild), flush=True)
    ins = oracle.make_inputs(B, T, H, N, 500 + T, with_state=True)
    if wild:
        ins[3][B - 1, T // 3:T // 3 + 20, 5:25] = 6.0
    dev, ref = cast_inputs(ins[:5], dtype)
    gyd, gyr = cast_inputs(ins[5:6], torch.float32)
    s0 = ins[6].float() * 3 if with_s0 else None
    gS = torch.randn(B, H, N, N, generator=torch.Generator().manual_seed(T)) if with_gs else None
    leaves = [x.clone().requires_grad_(True) for x in dev]
    s0_dev = s0.cuda().requires_grad_(True) if with_s0 else None
    op.algo = AUTO
    y, sT = op(*leaves, return_state=True, init_state=s0_dev)
    loss = (y * gyd[0]).sum()
    if with_gs:
        loss = loss + (sT * gS.cuda()).sum()
    got = torch.autograd.grad(loss, leaves + ([s0_dev] if with_s0 else []))
    torch.cuda.synchronize()
    want = oracle.backward_state_c(*ref, gyr[0], N, None if s0 is None else to_np(s0), None if gS is None else to_np(gS))
    y_ref, sT_ref = oracle.forward_c(*ref, N, None if s0 is None else to_np(s0))
    check_close("y", y.detach(), y_ref, torch.float32)
    check_close("sT", sT.detach(), sT_ref, torch.float32, is_grad=True)
    _check_grads(got[:5], want[:5], dtype)
    if with_s0:
        check_close("gs0", to_np(got[5]), want[5], torch.float32, is_grad=True)
    else:
        assert float(got[3][:, 0].abs().max()) == 0.0      # zero initial state: the first decay reaches nothing
    if not with_gs:
        assert float(got[3][:, -1].abs().max()) == 0.0
    # the same call on the per-timestep kernels agrees to fp32 rounding
    op.algo = SCAN
    leaves2 = [x.clone().requires_grad_(True) for x in dev]
    s0_2 = s0.cuda().requires_grad_(True) if with_s0 else None
    y2, sT2 = op(*leaves2, return_state=True, init_state=s0_2)
    loss2 = (y2 * gyd[0]).sum() + ((sT2 * gS.cuda()).sum() if with_gs else 0.0)
    got2 = torch.autograd.grad(loss2, leaves2 + ([s0_2] if with_s0 else []))
    torch.cuda.synchronize()
    tol = 2e-3 if dtype == torch.float16 else 5e-5
    for a_, b_ in zip(got, got2):
        assert float((a_.double() - b_.double()).abs().max()) <= tol * max(float(b_.double().abs().max()), 1e-30)


def test_decay_outside_the_reach_is_redone_exactly(op, oracle):
    # one pair decays by e^-4.5 per token over 40 tokens (a half-chunk sum of 72 > 40), another carries the
    # model's padding values (w = -1e9: decay exactly 1, with k = 0) and a decay of exactly 0 (w = 20): those
    # pairs take the per-timestep pass inside the same launches, the others stay on the chunk form
    def edit(ins):
        ins[3][0, 40:80, :64] = 1.5
        ins[3][1, 10:30, 64:128] = -1e9
        ins[1][1, 10:30, 64:128] = 0
        ins[3][1, 50, 64:128] = 20.0

    y, grads = _case(op, oracle, 2, 256, 3, 9, torch.float32, edit=edit)
    assert all(torch.isfinite(t).all() for t in [y] + grads)


def test_small_decay_sums_and_constant_inputs(op):
    # reference test_jax.py:12-16: r=k=v=u=1, w=-4 -> y_t = 64*(1 + (1-d^t)/(1-d)), d = exp(-exp(-4))
    B, T, C = 2, 512, 256
    one = torch.ones(B, T, C, device="cuda")
    op.algo = AUTO
    with torch.no_grad():
        y, _ = op(one, one, one, one * 0 - 4, torch.ones(C, device="cuda"))
    d = np.exp(-np.exp(-4.0))
    expect = 64 * (1 + (1 - d ** np.arange(T)) / (1 - d))
    got = to_np(y)
    assert got[0, 0, 0] == 64.0
    np.testing.assert_allclose(got[1, :, 77], expect, rtol=2e-5)


@pytest.mark.parametrize("dt", ["f32", "f16"])
def test_saved_and_recomputed_states_give_the_same_gradients(lib, oracle, dt):
    # wkv6_forward / wkv6_backward (the reference-shaped pair: a forward pass that only leaves the chunk states
    # comes first) against wkv6_forward_save / wkv6_backward_saved_sum: the same kernels on the same states,
    # bit for bit; y does not depend on whether the states are kept
    from rwkv_kernel import _native

    B, T, H = 3, 200, 2
    C = H * N
    code = _native.F32 if dt == "f32" else _native.F16
    ins = oracle.make_inputs(B, T, H, N, 33)
    dev, ref = cast_inputs(ins[:5], DTYPES[dt])
    gyd, gyr = cast_inputs(ins[5:6], torch.float32)
    r, k, v, w, u = dev
    gy = gyd[0]
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    n = lib.wkv6_saved_bytes(code, AUTO, B, T, C, H)
    assert n == lib.wkv6_backward_workspace_bytes_ex(code, AUTO, B, T, C, H) > 0
    res = []
    for mode in ("plain", "saved"):
        y = torch.empty(B, T, C, dtype=torch.float32, device="cuda")
        outs = [torch.empty(B, T, C, dtype=torch.float32, device="cuda") for _ in range(4)]
        gu = torch.empty(B, C, dtype=torch.float32, device="cuda")
        gus = torch.zeros(C, dtype=torch.float32, device="cuda")
        buf = torch.empty(n, dtype=torch.uint8, device="cuda")
        if mode == "plain":
            _native.check(lib.wkv6_forward(st, code, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y)))
            _native.check(lib.wkv6_backward(st, code, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                            *[P(o) for o in outs], P(gu), P(buf), n))
        else:
            _native.check(lib.wkv6_forward_save(st, code, AUTO, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), P(buf), n))
            _native.check(lib.wkv6_backward_saved_sum(st, code, AUTO, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                      *[P(o) for o in outs], P(gu), P(gus), P(buf), n))
        torch.cuda.synchronize()
        res.append([y] + outs + [gu, gus])
    for a, b in zip(res[0][:6], res[1][:6]):
        assert torch.equal(a, b)
    g_ref = oracle.backward_c(*ref, gyr[0], N)
    check_close("y", res[1][0], oracle.forward_c(*ref, N)[0], torch.float32)
    for name, g, gr in zip("gr gk gv gw".split(), res[1][1:5], g_ref):
        check_close(name, g, gr, torch.float32, is_grad=True)
    check_close("gu summed", to_np(res[1][6]).reshape(H, N), g_ref[4], torch.float32, is_grad=True)
    check_close("gu rows", to_np(res[1][5]).sum(0).reshape(H, N), g_ref[4], torch.float32, is_grad=True)


def test_fp16_inference_on_request_too(op, oracle):
    # a forward of fp16 tensors asked for as WKV6_ALGO_CHUNK has no bf16-operand form: it runs at full precision
    ins = oracle.make_inputs(2, 256, 2, N, 5)
    dev, ref = cast_inputs(ins[:5], torch.float16)
    outs = []
    for algo in (AUTO, CHUNK, SCAN):
        op.algo = algo
        with torch.no_grad():
            outs.append(op(*dev)[0])
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    y_ref, _ = oracle.forward_c(*ref, N)
    for y in outs:
        check_close("y", y, y_ref, torch.float32)


def test_c2_shape_fp32_vs_oracle(op, oracle):
    # B=8 T=1024 C=2048 H=32 with fp32 tensors: every output against the float64 oracle
    B, T, H = 8, 1024, 32
    print("C2 shape, fp32", flush=True)
    ins = oracle.make_inputs(B, T, H, N, 0)
    dev, ref = cast_inputs(ins[:5], torch.float32)
    gyd, gyr = cast_inputs(ins[5:6], torch.float32)
    y, grads = _fwd_bwd(op, dev, gyd[0], AUTO)
    check_close("y", y, oracle.forward_c(*ref, N)[0], torch.float32)
    _check_grads(grads, oracle.backward_c(*ref, gyr[0], N), torch.float32)


def test_random_shapes_against_the_oracle_and_the_per_timestep_kernels(op, oracle):
    # 40 random (B, T, H, dtype, kind) cases, some with a stretch of strong decay in one pair, through
    # WKV6_ALGO_AUTO and WKV6_ALGO_SCAN: each against the float64 oracle at the fp32 tolerances, and the two kernel
    # families against each other to fp32 rounding
    import random

    rng = random.Random(2024)

    def rel(a, b):
        return float((a.double() - b.double()).abs().max() / max(float(b.double().abs().max()), 1e-30))

    for case in range(40):
        B, H = rng.choice([1, 2, 3, 5, 9, 33]), rng.choice([1, 2, 3, 5, 8])
        T = rng.choice([64, 65, 95, 96, 97, 127, 128, 160, 333, 511, 1000])
        if B * H * T > 300000:
            T = 128
        dt = rng.choice([torch.float32, torch.float16])
        kind = rng.choice(["train", "train", "state", "infer"])
        g = torch.Generator().manual_seed(7000 + case)
        C = H * N
        r, k, v = [torch.randn(B, T, C, generator=g) for _ in range(3)]
        w = torch.rand(B, T, C, generator=g) * 7 - 6
        u = torch.randn(H, N, generator=g) * 0.5
        gy = torch.randn(B, T, C, generator=g).cuda()
        if rng.random() < 0.3:
            b0, h0, t0 = rng.randrange(B), rng.randrange(H), rng.randrange(T - 20)
            w[b0, t0:t0 + rng.choice([12, 20]), N * h0:N * h0 + N] = rng.choice([1.2, 2.0, 20.0])
        dev = [x.to(dt).cuda() for x in (r, k, v, w, u)]
        nrow = rng.choice([1, B])
        s0 = (torch.randn(nrow, H, N, N, generator=g) * 0.1).cuda()
        smap = [rng.randrange(nrow) for _ in range(B)]
        print("case %d B%d T%d H%d %s %s" % (case, B, T, H, dt, kind), flush=True)
        outs = {}
        for algo in (AUTO, SCAN):
            op.algo = algo
            if kind == "train":
                leaves = [x.clone().requires_grad_(True) for x in dev]
                y, _ = op(*leaves)
                y.backward(gy)
                outs[algo] = [y.detach()] + [x.grad for x in leaves]
            elif kind == "state":
                with torch.no_grad():
                    outs[algo] = list(op(*dev, return_state=True, init_state=s0, state_map=smap))
            else:
                with torch.no_grad():
                    outs[algo] = [op(*dev)[0]]
        torch.cuda.synchronize()
        ref = [to_np(x) for x in dev]
        if kind == "train":
            want = [oracle.forward_c(*ref, N)[0]] + list(oracle.backward_c(*ref, to_np(gy), N))
        elif kind == "state":
            want = list(oracle.forward_c(*ref, N, to_np(s0), smap))
        else:
            want = [oracle.forward_c(*ref, N)[0]]
        for algo in (AUTO, SCAN):
            for i, (got, w_) in enumerate(zip(outs[algo], want)):
                # (y is fp32 whatever the tensors are; fp16 gradients come back rounded to fp16)
                tol_dt = torch.float16 if (dt == torch.float16 and kind == "train" and i > 0) else torch.float32
                check_close("case %d algo %d output %d" % (case, algo, i), to_np(got).reshape(w_.shape), w_, tol_dt, is_grad=i > 0)
        tol = 2e-3 if dt == torch.float16 and kind == "train" else 2e-5   # (fp16 gradients come back rounded to fp16)
        for a, b in zip(outs[AUTO], outs[SCAN]):
            assert torch.isfinite(a.float()).all()
            assert rel(a, b) <= tol, (case, rel(a, b))
