"""wkv6_backward_static: the backward whose workspace is the library's own fixed device array (no
allocation in the call) against wkv6_backward with a caller-owned workspace, through the C ABI, on
two calls in a row -- the second on a smaller input, so that it runs over what the first left in
the shared array -- then a shape the array is too small for."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _pair(lib, native, B, T, H, dtype, seed):
    N = 64
    C = H * N
    code = {torch.bfloat16: native.BF16, torch.float32: native.F32}[dtype]
    g = torch.Generator().manual_seed(seed)
    r, k, v, gy = (torch.randn(B, T, C, generator=g).to(dtype).cuda() for _ in range(4))
    w = (torch.rand(B, T, C, generator=g) * 7.0 - 6.0).to(dtype).cuda()
    u = (torch.randn(H, N, generator=g) * 0.5).to(dtype).cuda()
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()

    def outs():
        return [torch.full((B, T, C), float("nan"), dtype=dtype, device="cuda") for _ in range(4)] + \
               [torch.full((B, C), float("nan"), dtype=dtype, device="cuda")]

    n = lib.wkv6_backward_workspace_bytes(code, B, T, C, H)
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device="cuda")
    want = outs()
    native.check(lib.wkv6_backward(st, code, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in want], P(ws), n))
    got = outs()

    def call():
        native.check(lib.wkv6_backward_static(st, code, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in got]))
        torch.cuda.synchronize()

    call()   # (the first call on a device looks the array's address up and sets the kernels' attributes)
    # the device's own count of free memory, which sees every allocation of the process, not only torch's
    free_before = torch.cuda.mem_get_info()[0]
    torch_before = torch.cuda.memory_allocated()
    for x in got:
        x.fill_(float("nan"))
    call()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == torch_before
    return got, want


def test_static_scratch_backward_equals_workspace_backward():
    from rwkv_kernel import _native

    lib = _native.load()
    torch.cuda.set_device(0)
    # first the largest shape the array holds (the benchmark's), then smaller ones on every kernel family
    for B, T, H, dtype, seed in ((8, 1024, 32, torch.bfloat16, 0), (3, 200, 2, torch.bfloat16, 1), (2, 200, 3, torch.float32, 3),
                                 (2, 77, 3, torch.float32, 2)):   # (fp32: the full-precision chunk form, then the per-timestep kernels)
        print("static scratch backward B%d T%d H%d %s" % (B, T, H, dtype), flush=True)
        assert lib.wkv6_backward_workspace_bytes(
            _native.BF16 if dtype == torch.bfloat16 else _native.F32, B, T, H * 64, H) <= _native.STATIC_SCRATCH_BYTES
        got, want = _pair(lib, _native, B, T, H, dtype, seed)
        for name, a, b in zip("gr gk gv gw gu".split(), got, want):
            assert bool(torch.isfinite(a.float()).all()), name
            assert torch.equal(a, b), "%s differs (max %g)" % (name, float((a.float() - b.float()).abs().max()))


def test_static_scratch_backward_takes_the_smaller_workspace_when_only_that_fits():
    # fp32 tensors at the benchmark's shape: the chunk states of the full-precision chunk form (128 MiB) do not
    # fit the array, the rows of the per-timestep kernels (64 MiB) do: the call runs those, bit for bit
    from rwkv_kernel import _native

    lib = _native.load()
    torch.cuda.set_device(0)
    B, T, H = 8, 1024, 32
    C = H * 64
    assert lib.wkv6_backward_workspace_bytes(_native.F32, B, T, C, H) > _native.STATIC_SCRATCH_BYTES
    n = lib.wkv6_backward_workspace_bytes_ex(_native.F32, _native.ALGO_SCAN, B, T, C, H)
    assert n <= _native.STATIC_SCRATCH_BYTES
    g = torch.Generator().manual_seed(5)
    r, k, v, gy = (torch.randn(B, T, C, generator=g).cuda() for _ in range(4))
    w = (torch.rand(B, T, C, generator=g) * 7.0 - 6.0).cuda()
    u = (torch.randn(H, 64, generator=g) * 0.5).cuda()
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    outs = lambda: [torch.empty(B, T, C, device="cuda") for _ in range(4)] + [torch.empty(B, C, device="cuda")]
    want, got = outs(), outs()
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    _native.check(lib.wkv6_backward_ex(st, _native.F32, _native.ALGO_SCAN, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                       *[P(x) for x in want], P(ws), n))
    _native.check(lib.wkv6_backward_static(st, _native.F32, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in got]))
    torch.cuda.synchronize()
    for name, a, b in zip("gr gk gv gw gu".split(), got, want):
        assert torch.equal(a, b), name


def test_static_scratch_backward_refuses_what_does_not_fit():
    from rwkv_kernel import _native

    lib = _native.load()
    B, T, H = 8, 2048, 32   # twice the benchmark's tokens: 128 MiB of workspace
    C = H * 64
    assert lib.wkv6_backward_workspace_bytes(_native.BF16, B, T, C, H) > _native.STATIC_SCRATCH_BYTES
    x = torch.zeros(16, dtype=torch.bfloat16, device="cuda")   # never dereferenced: the size check comes first
    p = x.data_ptr()
    rc = lib.wkv6_backward_static(None, _native.BF16, B, T, C, H, *([p] * 11))
    assert rc == 3 and b"workspace" in lib.wkv6_status_string(rc)


def test_static_scratch_backward_replays_in_a_hip_graph():
    """The call captured once into a graph (it allocates nothing and enqueues on the given stream only) and
    replayed on changed inputs, with eager work in between: every replay equals wkv6_backward on the same
    inputs."""
    from rwkv_kernel import _native

    lib = _native.load()
    torch.cuda.set_device(0)
    B, T, H, N = 4, 256, 8, 64
    C = H * N
    g = torch.Generator().manual_seed(31)
    src = [torch.randn(B, T, C, generator=g) for _ in range(4)] + [torch.rand(B, T, C, generator=g) * 7.0 - 6.0]
    r, k, v, gy, w = (x.to(torch.bfloat16).cuda() for x in src)
    u = (torch.randn(H, N, generator=g) * 0.5).to(torch.bfloat16).cuda()
    got = [torch.empty(B, T, C, dtype=torch.bfloat16, device="cuda") for _ in range(4)] + [torch.empty(B, C, dtype=torch.bfloat16, device="cuda")]
    P = lambda t: t.data_ptr()

    def step():
        st = torch.cuda.current_stream().cuda_stream
        _native.check(lib.wkv6_backward_static(st, _native.BF16, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in got]))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                      # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    n = lib.wkv6_backward_workspace_bytes(_native.BF16, B, T, C, H)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    for rep in range(3):
        # changed inputs (in place: the graph holds the addresses), eager work between the replays
        v.copy_((torch.randn(B, T, C, generator=g)).to(torch.bfloat16))
        gy.copy_((torch.randn(B, T, C, generator=g)).to(torch.bfloat16))
        for x in got:
            x.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = [torch.empty_like(x) for x in got]
        st = torch.cuda.current_stream().cuda_stream
        _native.check(lib.wkv6_backward(st, _native.BF16, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in want], P(ws), n))
        torch.cuda.synchronize()
        for name, a, b in zip("gr gk gv gw gu".split(), got, want):
            assert torch.equal(a, b), (rep, name)
