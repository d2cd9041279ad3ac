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
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    native.check(lib.wkv6_backward_static(st, code, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy), *[P(x) for x in got]))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return got, want


def test_static_scratch_backward_equals_workspace_backward():
    from rwkv_kernel import _native

    lib = _native.load()
    torch.cuda.set_device(0)
    # first the largest shape the array holds (the benchmark's), then smaller ones on both kernel families
    for B, T, H, dtype, seed in ((8, 1024, 32, torch.bfloat16, 0), (3, 200, 2, torch.bfloat16, 1), (2, 77, 3, torch.float32, 2)):
        print("static scratch backward B%d T%d H%d %s" % (B, T, H, dtype), flush=True)
        assert lib.wkv6_backward_workspace_bytes(
            _native.BF16 if dtype == torch.bfloat16 else _native.F32, B, T, H * 64, H) <= _native.STATIC_SCRATCH_BYTES
        got, want = _pair(lib, _native, B, T, H, dtype, seed)
        for name, a, b in zip("gr gk gv gw gu".split(), got, want):
            assert bool(torch.isfinite(a.float()).all()), name
            assert torch.equal(a, b), "%s differs (max %g)" % (name, float((a.float() - b.float()).abs().max()))


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
