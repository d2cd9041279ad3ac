"""The input side of the time-mix layer (token shift and the five low-rank mixers, rwkv6_model.py:134-146)
on the GPU, through the C ABI, against the float64 restatement in oracle/ on the same bf16-rounded
inputs; the gradients against torch.autograd through that restatement in float64."""
import numpy as np
import pytest
import torch

from _util import check_close, rel_inf, rel_l2, to_np

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16

# (B, T, C, R): token counts that are no multiple of the 16-token MFMA block or the 128-token
# workgroup, T = 1 (no previous token anywhere), C that is no multiple of a workgroup's 256 channels
SHAPES = [(2, 64, 128, 32), (3, 37, 64, 32), (5, 1, 192, 32), (1, 300, 320, 64), (2, 129, 256, 64), (8, 256, 512, 32)]


@pytest.fixture(scope="module")
def lib():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from rwkv_kernel import _native
    return _native.load()


def _inputs(B, T, C, R, seed):
    """bf16-rounded tensors on the GPU and their float64 values."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, C, generator=g)
    mix_x = torch.rand(C, generator=g)
    a = torch.randn(5 * R, C, generator=g) / C ** 0.5
    w2t = torch.randn(5, C, R, generator=g) / R ** 0.5
    bias = torch.rand(5, C, generator=g)
    dev = dict(x=x.to(BF16).cuda(), mix_x=mix_x.cuda(), a=a.to(BF16).cuda(), w2t=w2t.to(BF16).cuda(), bias=bias.cuda())
    ref = {k: to_np(v) for k, v in dev.items()}
    return dev, ref


def _stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("B,T,C,R", SHAPES)
def test_forward_kernels(lib, oracle, B, T, C, R):
    from rwkv_kernel import _native
    print("shift_mix forward B=%d T=%d C=%d R=%d" % (B, T, C, R), flush=True)
    assert lib.wkv6_shift_mix_supported(_native.BF16, C, R) == 1
    dev, ref = _inputs(B, T, C, R, 10 * T + R)
    x_mix = torch.empty_like(dev["x"])
    _native.check(lib.wkv6_shift_mix_x(_stream(), _native.BF16, B, T, C, dev["x"].data_ptr(), dev["mix_x"].data_ptr(), x_mix.data_ptr()))
    want_mix, _, _ = oracle.shift_mix_np(ref["x"], ref["mix_x"], ref["a"], ref["w2t"], ref["bias"])
    check_close("x_mix", x_mix, want_mix, BF16)
    # the second kernel takes h as the caller computed it: feed both sides the same bf16 h
    g = torch.Generator().manual_seed(T)
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(BF16).cuda()
    outs = [torch.full((B, T, C), float("nan"), dtype=BF16, device="cuda") for _ in range(5)]
    _native.check(lib.wkv6_shift_mix_five(_stream(), _native.BF16, B, T, C, R, dev["x"].data_ptr(), h.data_ptr(), dev["w2t"].data_ptr(),
                                          dev["bias"].data_ptr(), *[o.data_ptr() for o in outs]))
    torch.cuda.synchronize()
    x, hh = ref["x"], to_np(h)
    xx = np.concatenate([np.zeros((B, 1, C)), x[:, :-1]], 1) - x
    for s in range(5):
        want = x + xx * (hh[:, :, s] @ ref["w2t"][s].T + ref["bias"][s])
        check_close("out%d" % s, outs[s], want, BF16)
    # and the whole forward the way the operator object runs it (its own GEMM and tanh in between)
    import rwkv_kernel
    op = rwkv_kernel.RWKVKernelOperator(64, 4096)
    got = op.shift_mix(dev["x"], dev["mix_x"], dev["a"], dev["w2t"], dev["bias"])
    _, _, want = oracle.shift_mix_np(ref["x"], ref["mix_x"], ref["a"], ref["w2t"], ref["bias"])
    for s in range(5):
        check_close("x_s%d" % s, got[s], want[s], BF16)


@pytest.mark.parametrize("B,T,C,R", SHAPES)
def test_backward_kernels(lib, B, T, C, R):
    """wkv6_shift_mix_five_backward and wkv6_shift_mix_x_backward one at a time against the formulas'
    autograd in float64 (h and gxm are inputs here, as they are for the kernels)."""
    from rwkv_kernel import _native
    print("shift_mix backward kernels B=%d T=%d C=%d R=%d" % (B, T, C, R), flush=True)
    dev, ref = _inputs(B, T, C, R, 20 * T + R)
    g = torch.Generator().manual_seed(T + 1)
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(BF16).cuda()
    gouts = [torch.randn(B, T, C, generator=g).to(BF16).cuda() for _ in range(5)]
    gxm = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    # float64 autograd of  L = sum_s <x_s, g_s> + <x_mix, gxm>  with xx treated as its own leaf for gxx
    x = torch.tensor(ref["x"], requires_grad=True)
    mix = torch.tensor(ref["mix_x"], requires_grad=True)
    coef_leaf = [(torch.tensor(to_np(h))[:, :, s] @ torch.tensor(ref["w2t"][s]).T + torch.tensor(ref["bias"][s])).requires_grad_(True)
                 for s in range(5)]
    xx = (torch.cat([torch.zeros(B, 1, C, dtype=torch.float64), x[:, :-1]], 1) - x)
    xx_leaf = xx.detach().requires_grad_(True)
    loss5 = sum(((x.detach() + xx_leaf * coef_leaf[s]) * gouts[s].double().cpu()).sum() for s in range(5))
    loss5.backward()
    want_gxx = xx_leaf.grad.numpy()
    want_gcoef = np.stack([c.grad.numpy() for c in coef_leaf])
    want_gp = sum(to_np(go) for go in gouts) - want_gxx
    plane = B * T * C + 128 * (T % 2)        # planes back to back, or 256 bytes apart
    gcoef = torch.full((5 * plane,), float("nan"), dtype=BF16, device="cuda").as_strided((5, B * T, C), (plane, C, 1))
    gp, gxx = torch.empty_like(dev["x"]), torch.empty_like(dev["x"])
    _native.check(lib.wkv6_shift_mix_five_backward(
        _stream(), _native.BF16, B, T, C, R, dev["x"].data_ptr(), h.data_ptr(), dev["w2t"].data_ptr(), dev["bias"].data_ptr(),
        *[go.data_ptr() for go in gouts], gcoef.data_ptr(), plane, gp.data_ptr(), gxx.data_ptr()))
    torch.cuda.synchronize()
    check_close("gcoef", gcoef.reshape(5, B, T, C), want_gcoef, BF16, is_grad=True)
    check_close("gxx", gxx, want_gxx, BF16, is_grad=True)
    check_close("gp", gp, want_gp, BF16, is_grad=True)
    # second kernel: all of x's gradient, with gp and gxx as the first kernel wrote them (bf16)
    coefs = [c.detach() for c in coef_leaf]
    total = sum(((x + xx * coefs[s]) * gouts[s].double().cpu()).sum() for s in range(5)) + ((x + xx * mix) * gxm.double().cpu()).sum()
    total.backward()
    gx = torch.empty_like(dev["x"])
    gmix = torch.full((C,), 7.0, device="cuda")          # (the call zeroes the sum itself)
    _native.check(lib.wkv6_shift_mix_x_backward(_stream(), _native.BF16, B, T, C, dev["x"].data_ptr(), dev["mix_x"].data_ptr(),
                                                gp.data_ptr(), gxx.data_ptr(), gxm.data_ptr(), gx.data_ptr(), gmix.data_ptr()))
    torch.cuda.synchronize()
    check_close("gx", gx, x.grad.numpy(), BF16, is_grad=True)
    check_close("gmix_x", gmix.cpu().double().numpy(), mix.grad.numpy(), torch.float32, is_grad=True)


def test_backward_kernels_full_size(lib):
    """The two backward kernels at the training benchmark's layer shape (B=8, T=1024, C=2048, rank 32)
    with random coefficients: every output of one batch row (a row's tokens only see that row) against
    the formulas' autograd in float64, and gmix_x -- a sum over all rows and tokens -- against its
    float64 value over everything."""
    from rwkv_kernel import _native
    B, T, C, R, row = 8, 1024, 2048, 32, 5
    print("shift_mix backward kernels, full size", flush=True)
    dev, ref = _inputs(B, T, C, R, 4242)
    g = torch.Generator().manual_seed(4243)
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(BF16).cuda()
    gouts = [torch.randn(B, T, C, generator=g).to(BF16).cuda() for _ in range(5)]
    gxm = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    plane = B * T * C
    gcoef = torch.full((5, B * T, C), float("nan"), dtype=BF16, device="cuda")
    gp, gxx, gx = (torch.full_like(dev["x"], float("nan")) for _ in range(3))
    gmix = torch.full((C,), 7.0, device="cuda")
    _native.check(lib.wkv6_shift_mix_five_backward(
        _stream(), _native.BF16, B, T, C, R, dev["x"].data_ptr(), h.data_ptr(), dev["w2t"].data_ptr(), dev["bias"].data_ptr(),
        *[go.data_ptr() for go in gouts], gcoef.data_ptr(), plane, gp.data_ptr(), gxx.data_ptr()))
    _native.check(lib.wkv6_shift_mix_x_backward(_stream(), _native.BF16, B, T, C, dev["x"].data_ptr(), dev["mix_x"].data_ptr(),
                                                gp.data_ptr(), gxx.data_ptr(), gxm.data_ptr(), gx.data_ptr(), gmix.data_ptr()))
    torch.cuda.synchronize()
    # one row in float64
    x = torch.tensor(ref["x"][row:row + 1], requires_grad=True)
    mix = torch.tensor(ref["mix_x"], requires_grad=True)
    hh = torch.tensor(to_np(h[row:row + 1]))
    go = [torch.tensor(to_np(t[row:row + 1])) for t in gouts]
    coef_leaf = [(hh[:, :, s] @ torch.tensor(ref["w2t"][s]).T + torch.tensor(ref["bias"][s])).requires_grad_(True) for s in range(5)]
    xx = torch.cat([torch.zeros(1, 1, C, dtype=torch.float64), x[:, :-1]], 1) - x
    xx_leaf = xx.detach().requires_grad_(True)
    sum(((x.detach() + xx_leaf * coef_leaf[s]) * go[s]).sum() for s in range(5)).backward()
    want_gxx = xx_leaf.grad.numpy()
    check_close("gcoef", gcoef.view(5, B, T, C)[:, row:row + 1], np.stack([c.grad.numpy() for c in coef_leaf]), BF16, is_grad=True)
    check_close("gxx", gxx[row:row + 1], want_gxx, BF16, is_grad=True)
    check_close("gp", gp[row:row + 1], sum(t.numpy() for t in go) - want_gxx, BF16, is_grad=True)
    coefs = [c.detach() for c in coef_leaf]
    (sum(((x + xx * coefs[s]) * go[s]).sum() for s in range(5)) + ((x + xx * mix) * torch.tensor(to_np(gxm[row:row + 1]))).sum()).backward()
    check_close("gx", gx[row:row + 1], x.grad.numpy(), BF16, is_grad=True)
    # gmix_x over everything: sum_{b,t} gxm * xx
    xa = ref["x"]
    xxa = np.concatenate([np.zeros((B, 1, C)), xa[:, :-1]], 1) - xa
    check_close("gmix_x", gmix.cpu().double().numpy(), (to_np(gxm) * xxa).sum((0, 1)), torch.float32, is_grad=True)
    for t in (gcoef, gp, gxx, gx):
        assert bool(torch.isfinite(t.float()).all())


@pytest.mark.parametrize("B,T,C,R", [(2, 64, 128, 32), (3, 37, 64, 32), (1, 300, 320, 64), (4, 128, 512, 32)])
def test_autograd_through_the_operator_object(oracle, B, T, C, R):
    """op.shift_mix end to end, gradients of all five arguments, against float64 autograd through the
    restated forward.  The chain holds three bf16 GEMMs of torch between the kernels; the tolerance
    is the 16-bit one on the l2 norm and three times that on the largest single element."""
    import rwkv_kernel
    op = rwkv_kernel.RWKVKernelOperator(64, 4096)
    print("shift_mix autograd B=%d T=%d C=%d R=%d" % (B, T, C, R), flush=True)
    dev, ref = _inputs(B, T, C, R, 30 * T + R)
    g = torch.Generator().manual_seed(T + 2)
    gouts = [torch.randn(B, T, C, generator=g).to(BF16).cuda() for _ in range(5)]
    leaves = {k: v.clone().requires_grad_(True) for k, v in dev.items()}
    outs = op.shift_mix(leaves["x"], leaves["mix_x"], leaves["a"], leaves["w2t"], leaves["bias"])
    torch.autograd.backward(outs, gouts)
    torch.cuda.synchronize()
    t = {k: torch.tensor(v, requires_grad=True) for k, v in ref.items()}
    x = t["x"]
    xx = torch.cat([torch.zeros(B, 1, C, dtype=torch.float64), x[:, :-1]], 1) - x
    x_mix = x + xx * t["mix_x"]
    hh = torch.tanh(x_mix @ t["a"].T).view(B, T, 5, R)
    loss = 0.0
    for s in range(5):
        want = x + xx * (hh[:, :, s] @ t["w2t"][s].T + t["bias"][s])
        # forward agrees with the numpy restatement (which the CPU tests pin) and with the kernels
        loss = loss + (want * gouts[s].double().cpu()).sum()
        check_close("x_s%d" % s, outs[s], want.detach().numpy(), BF16)
    _, _, want_np = oracle.shift_mix_np(ref["x"], ref["mix_x"], ref["a"], ref["w2t"], ref["bias"])
    assert np.abs(want_np[4] - want.detach().numpy()).max() < 1e-12
    loss.backward()
    for k in ("x", "mix_x", "a", "w2t", "bias"):
        got, want = to_np(leaves[k].grad), t[k].grad.numpy()
        e1, e2 = rel_inf(got, want), rel_l2(got, want)
        print("  grad %-5s rel-inf %.2e rel-l2 %.2e" % (k, e1, e2), flush=True)
        assert e2 <= 1e-2 and e1 <= 3e-2, (k, e1, e2)


def test_unsupported_shapes_are_refused(lib):
    from rwkv_kernel import _native
    assert lib.wkv6_shift_mix_supported(_native.BF16, 128, 8) == 0        # rank below one MFMA's depth
    assert lib.wkv6_shift_mix_supported(_native.BF16, 96, 32) == 0        # channels no multiple of 64
    assert lib.wkv6_shift_mix_supported(_native.F32, 128, 32) == 0
    x = torch.zeros(1, 4, 128, dtype=BF16, device="cuda")
    m = torch.zeros(128, device="cuda")
    rc = lib.wkv6_shift_mix_x(_stream(), _native.F32, 1, 4, 128, x.data_ptr(), m.data_ptr(), x.data_ptr())
    assert rc == 2          # WKV6_ERR_UNSUPPORTED
    rc = lib.wkv6_shift_mix_x(_stream(), _native.BF16, 1, 4, 128, None, m.data_ptr(), x.data_ptr())
    assert rc == 1          # WKV6_ERR_ARG


def test_full_size_known_answers(lib):
    """At the benchmark's layer shape (B=8, T=1024, C=2048, rank 32), where a float64 reference of
    everything is too slow: cases whose exact answer needs no arithmetic.  Coefficient 0 (W = 0,
    bias = 0) must return x bit for bit in all five outputs; coefficient 1 must return the previous
    token (x + (prev - x) in fp32: to one bf16 rounding plus 2^-23 of |x|; exactly zero at the start
    of every sequence); and with coefficient 1 the backward
    kernel's gp = sum_s g_s - gxx must be exactly zero wherever gxx, five bf16 values summed in
    fp32, is itself a bf16 number -- checked through gp + gxx = sum_s g_s to one rounding."""
    from rwkv_kernel import _native
    B, T, C, R = 8, 1024, 2048, 32
    g = torch.Generator().manual_seed(77)
    x = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(BF16).cuda()
    zero_w = torch.zeros(5, C, R, dtype=BF16, device="cuda")
    outs = [torch.full((B, T, C), float("nan"), dtype=BF16, device="cuda") for _ in range(5)]

    def five(bias):
        _native.check(lib.wkv6_shift_mix_five(_stream(), _native.BF16, B, T, C, R, x.data_ptr(), h.data_ptr(), zero_w.data_ptr(),
                                              bias.data_ptr(), *[o.data_ptr() for o in outs]))
        torch.cuda.synchronize()

    five(torch.zeros(5, C, device="cuda"))
    assert all(torch.equal(o, x) for o in outs)
    five(torch.ones(5, C, device="cuda"))
    prev = torch.cat([torch.zeros(B, 1, C, dtype=BF16, device="cuda"), x[:, :-1]], 1)
    slack = 2.0 ** -23 * float(x.float().abs().max())
    for o in outs:
        assert torch.allclose(o.float(), prev.float(), rtol=2.0 ** -8, atol=slack)
        assert float(o[:, 0].float().abs().max()) == 0.0
    # x_mix with mix_x = 1 is the previous token as well, with mix_x = 0 it is x
    x_mix = torch.empty_like(x)
    for val, want in ((1.0, prev), (0.0, x)):
        m = torch.full((C,), val, device="cuda")
        _native.check(lib.wkv6_shift_mix_x(_stream(), _native.BF16, B, T, C, x.data_ptr(), m.data_ptr(), x_mix.data_ptr()))
        torch.cuda.synchronize()
        assert torch.allclose(x_mix.float(), want.float(), rtol=2.0 ** -8, atol=slack)
    assert torch.equal(x_mix, x)                       # (mix_x = 0: bit for bit)
    # backward with coefficient 1: gcoef_s = g_s * xx, gxx = sum_s g_s, gp = 0 up to gxx's own rounding
    gouts = [torch.randn(B, T, C, generator=g).to(BF16).cuda() for _ in range(5)]
    plane = B * T * C
    gcoef = torch.empty(5, B * T, C, dtype=BF16, device="cuda")
    gp, gxx = torch.empty_like(x), torch.empty_like(x)
    _native.check(lib.wkv6_shift_mix_five_backward(
        _stream(), _native.BF16, B, T, C, R, x.data_ptr(), h.data_ptr(), zero_w.data_ptr(), torch.ones(5, C, device="cuda").data_ptr(),
        *[go.data_ptr() for go in gouts], gcoef.data_ptr(), plane, gp.data_ptr(), gxx.data_ptr()))
    torch.cuda.synchronize()
    total = sum(go.float() for go in gouts)
    assert torch.equal(gxx, total.to(BF16))
    assert float(gp.float().abs().max()) == 0.0       # sum - gxx in fp32, before gxx is rounded: exactly zero
    xx = prev.float() - x.float()
    for s in range(5):
        assert torch.equal(gcoef[s].view(B, T, C), (gouts[s].float() * xx).to(BF16))


def test_calls_replay_in_a_hip_graph(lib):
    """The four calls captured once into a graph (they allocate nothing, enqueue on the given stream
    only and clear gmix_x with a kernel of their own) and replayed with eager work in between: every
    replay reproduces the eager results (bit for bit, except gmix_x whose atomic sums may come in
    another order)."""
    from rwkv_kernel import _native
    B, T, C, R = 3, 200, 320, 32
    dev, _ = _inputs(B, T, C, R, 5)
    g = torch.Generator().manual_seed(6)
    h = torch.tanh(torch.randn(B, T, 5, R, generator=g)).to(BF16).cuda()
    gouts = [torch.randn(B, T, C, generator=g).to(BF16).cuda() for _ in range(5)]
    gxm = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    res = {n: torch.empty_like(dev["x"]) for n in ("x_mix", "o0", "o1", "o2", "o3", "o4", "gp", "gxx", "gx")}
    res["gcoef"] = torch.empty(5, B * T, C, dtype=BF16, device="cuda")
    res["gmix"] = torch.empty(C, device="cuda")
    P = lambda t: t.data_ptr()

    def step():
        st = torch.cuda.current_stream().cuda_stream
        _native.check(lib.wkv6_shift_mix_x(st, _native.BF16, B, T, C, P(dev["x"]), P(dev["mix_x"]), P(res["x_mix"])))
        _native.check(lib.wkv6_shift_mix_five(st, _native.BF16, B, T, C, R, P(dev["x"]), P(h), P(dev["w2t"]), P(dev["bias"]),
                                              *[P(res["o%d" % s]) for s in range(5)]))
        _native.check(lib.wkv6_shift_mix_five_backward(st, _native.BF16, B, T, C, R, P(dev["x"]), P(h), P(dev["w2t"]), P(dev["bias"]),
                                                       *[P(go) for go in gouts], P(res["gcoef"]), B * T * C, P(res["gp"]), P(res["gxx"])))
        _native.check(lib.wkv6_shift_mix_x_backward(st, _native.BF16, B, T, C, P(dev["x"]), P(dev["mix_x"]), P(res["gp"]), P(res["gxx"]),
                                                    P(gxm), P(res["gx"]), P(res["gmix"])))

    step()
    torch.cuda.synchronize()
    eager = {n: t.clone() for n, t in res.items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                      # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in res.values():
            t.fill_(float("nan"))   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for n, t in res.items():
            if n == "gmix":
                assert torch.allclose(t, eager[n], rtol=1e-5, atol=1e-5), (rep, n)
            else:
                assert torch.equal(t, eager[n]), (rep, n)


@pytest.mark.parametrize("B,T,C", [(2, 64, 128), (3, 37, 64), (5, 1, 192), (1, 300, 320)])
def test_fixed_mix_on_its_own(B, T, C):
    """op.shift_mix_x: x + xx * mix and its gradients (the backward kernel with no gp / gxx) against
    float64 autograd."""
    import rwkv_kernel
    op = rwkv_kernel.RWKVKernelOperator(64, 4096)
    g = torch.Generator().manual_seed(40 + T)
    x = torch.randn(B, T, C, generator=g).to(BF16).cuda().requires_grad_(True)
    mix = torch.rand(C, generator=g).cuda().requires_grad_(True)
    gout = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    out = op.shift_mix_x(x, mix)
    out.backward(gout)
    torch.cuda.synchronize()
    xr = x.detach().double().cpu().requires_grad_(True)
    mr = mix.detach().double().cpu().requires_grad_(True)
    xx = torch.cat([torch.zeros(B, 1, C, dtype=torch.float64), xr[:, :-1]], 1) - xr
    want = xr + xx * mr
    want.backward(gout.double().cpu())
    check_close("x_mix", out, want.detach().numpy(), BF16)
    check_close("gx", x.grad, xr.grad.numpy(), BF16, is_grad=True)
    check_close("gmix", mix.grad.double().cpu().numpy(), mr.grad.numpy(), torch.float32, is_grad=True)
