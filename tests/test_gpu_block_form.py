"""The block-form MFMA kernels (32-token blocks scaled from the block middle; taken for bf16 tensors with
T a multiple of 64 and more than half as many (batch, head) pairs as the chip has compute units; the
forward also takes several pairs per workgroup) through the C ABI and the torch binding against the float64
oracle: shapes at the edges of their range, states in and out of the forward, decay beyond the scaled
operands' range, and the mixing of either form's forward with either form's backward."""
import numpy as np
import pytest
import torch

from _util import cast_inputs, check_close, check_composite, to_np

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
CHUNK = 2
N = 64


@pytest.fixture(scope="module")
def op():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import rwkv_kernel

    return rwkv_kernel.RWKVKernelOperator(N, 4096)


def _pairs_in_range(B, H):
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    return cus // 2 < B * H <= cus


def _several_pairs_per_workgroup(B, H):
    # more pairs than compute units: one workgroup per compute unit (rounded down to a multiple of H) runs
    # its pairs back to back through one pipeline
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    grid = cus // H * H
    return B * H > cus and grid * 10 >= cus * 9 and -(-B * H // grid) <= 64


def _fwd_bwd(op, ins, algo=CHUNK):
    dev, ref = cast_inputs(ins[:5], BF16)
    gy_dev, gy_ref = cast_inputs(ins[5:6], BF16)
    op.algo = algo
    leaves = [x.clone().requires_grad_(True) for x in dev]
    y, _ = op(*leaves)
    y.backward(gy_dev[0])
    torch.cuda.synchronize()
    return y, [x.grad for x in leaves], ref, gy_ref[0]


def _check(oracle, y, grads, ref, gy_ref):
    check_close("y", y, oracle.forward_c(*ref, N)[0], BF16)
    for name, g, want in zip("gr gk gv gw gu".split(), grads, oracle.backward_c(*ref, gy_ref, N)):
        check_close(name, to_np(g).reshape(want.shape), want, BF16, is_grad=True)
    # the gradient of the first and of the last decay of a sequence is zero by definition
    assert float(grads[3][:, 0].float().abs().max()) == 0.0 and float(grads[3][:, -1].float().abs().max()) == 0.0


# (B, T, H): one visit, two visits, an odd number of visits, the smallest and the largest pair counts of
# the range on a 256-CU chip, pairs that are no multiple of the heads of a workgroup row
@pytest.mark.parametrize("B,T,H", [(129, 64, 1), (256, 64, 1), (4, 128, 64), (43, 192, 3), (5, 320, 32), (131, 128, 1),
                                   (16, 512, 16), (2, 2048, 96)])
def test_block_form_fwd_bwd(op, oracle, B, T, H):
    assert _pairs_in_range(B, H) and T % 64 == 0, "shape outside the block form's range on this chip"
    print("block form B=%d T=%d H=%d" % (B, T, H), flush=True)
    y, grads, ref, gy_ref = _fwd_bwd(op, oracle.make_inputs(B, T, H, N, 500 + T + H))
    _check(oracle, y, grads, ref, gy_ref)


# More pairs than compute units.  (B, T, H): one chunk per pair (the pipeline's start spans three pairs), pairs
# that do not fill the last round of workgroups, a head count that does not divide the compute units (grid 240),
# many pairs per workgroup
@pytest.mark.parametrize("B,T,H", [(40, 64, 32), (75, 128, 4), (13, 192, 40), (300, 64, 8), (33, 256, 32)])
def test_block_form_several_pairs_per_workgroup(op, oracle, B, T, H):
    assert _several_pairs_per_workgroup(B, H) and T % 64 == 0
    print("block form, several pairs per workgroup B=%d T=%d H=%d" % (B, T, H), flush=True)
    y, grads, ref, gy_ref = _fwd_bwd(op, oracle.make_inputs(B, T, H, N, 700 + T + H))
    _check(oracle, y, grads, ref, gy_ref)


def test_block_form_several_pairs_state_in_out_and_fallback(op, oracle):
    """Several pairs per workgroup with an initial state through a state map and the final state out; pairs in the
    first, a middle and the last position of their workgroup leave the scaled operands' range and are redone
    exactly after the workgroup's last pair."""
    B, T, H, nstate = 40, 128, 32, 9
    assert _several_pairs_per_workgroup(B, H)
    ins = oracle.make_inputs(B, T, H, N, 91, with_state=True)
    ins[3][0, 10:30, 64:128] = 6.0        # batch row 0, head 1: first pair of its workgroup
    ins[3][17, 70:90, 0:64] = 6.0         # a middle one
    ins[3][39, 100:120, 31 * 64:] = 6.0   # the last
    dev, ref = cast_inputs(ins[:5], BF16)
    op.algo = CHUNK
    for sdt in (BF16, torch.float32):
        s_dev, s_ref = cast_inputs([ins[6][:nstate]], sdt)
        smap = [(5 * i + 2) % nstate for i in range(B)]
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
        torch.cuda.synchronize()
        y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
        check_close("y", y, y_ref, BF16)
        check_close("sT", sT, sT_ref, BF16)


def test_block_form_several_pairs_fallback_in_the_backward(op, oracle):
    """Forward and backward with several pairs per workgroup, of which the first, a middle and the last one of
    a workgroup are redone exactly: every gradient, and gu summed over the batch (the chunked pairs' rows
    added up inside the kernel as they are stored, the redone pairs' rows read back)."""
    B, T, H = 40, 128, 32
    assert _several_pairs_per_workgroup(B, H)
    ins = oracle.make_inputs(B, T, H, N, 93)
    ins[3][0, 10:30, 64:128] = 6.0
    ins[3][17, 70:90, 0:64] = 6.0
    ins[3][39, 100:120, 31 * 64:] = 6.0
    ins[3][39, 5:25, 0:64] = 6.0
    y, grads, ref, gy_ref = _fwd_bwd(op, ins)
    _check(oracle, y, grads, ref, gy_ref)


def test_block_form_extreme_decay(op, oracle):
    """Pairs whose decay leaves the scaled operands' range are redone with the exact per-timestep code inside
    the same launch (forward and backward decide alike); decay exactly 0 and exactly 1; a 16-token stretch
    just inside the range across a block boundary and across a chunk boundary."""
    B, T, H = 5, 256, 32
    assert _pairs_in_range(B, H)
    ins = oracle.make_inputs(B, T, H, N, 53)
    w = ins[3]
    w[1, 40:60, 70:90] = 6.0          # exp(6) = 403 per step: far beyond the limit (pair (1, 1))
    w[0, 5, 3] = 20.0                 # decay exactly 0
    w[0, 90:100] = -1e9               # decay exactly 1
    w[2, 24:40, 128:192] = 1.3        # 16 tokens of exp(1.3) = 3.67: sum 58.7 < 64, across the block middle ...
    w[3, 56:72, 0:64] = 1.3           # ... and across a chunk boundary
    y, grads, ref, gy_ref = _fwd_bwd(op, ins)
    _check(oracle, y, grads, ref, gy_ref)


@pytest.mark.parametrize("B,T,H,nstate", [(5, 256, 32, 5), (130, 128, 1, 7), (3, 64, 64, 2)])
def test_block_form_state_in_out(op, oracle, B, T, H, nstate):
    """The forward with an initial state (shared through a state map), final state out, bf16 and fp32 states."""
    assert _pairs_in_range(B, H)
    ins = oracle.make_inputs(max(B, nstate), T, H, N, 61 + B, with_state=True)
    dev, ref = cast_inputs([x[:B] for x in ins[:4]] + [ins[4]], BF16)
    op.algo = CHUNK
    for sdt in (BF16, torch.float32):
        s_dev, s_ref = cast_inputs([ins[6][:nstate]], sdt)
        smap = [(3 * i + 1) % nstate for i in range(B)]
        y, sT = op(*dev, return_state=True, init_state=s_dev[0], state_map=smap)
        torch.cuda.synchronize()
        y_ref, sT_ref = oracle.forward_c(*ref, N, s_ref[0], smap)
        check_close("y", y, y_ref, BF16)
        check_close("sT", sT, sT_ref, BF16)
    y0, s0 = op(*dev, return_state=True)
    torch.cuda.synchronize()
    y_ref, s_ref0 = oracle.forward_c(*ref, N)
    check_close("y from zero", y0, y_ref, BF16)
    check_close("sT from zero", s0, s_ref0, BF16)


def test_block_form_chunks_continue_each_other(op, oracle):
    """A sequence cut in two with the state handed across gives the uncut y and final state."""
    B, T, H = 5, 512, 32
    ins = oracle.make_inputs(B, T, H, N, 71)
    dev, ref = cast_inputs(ins[:5], BF16)
    op.algo = CHUNK
    first = [x[:, :192].contiguous() for x in dev[:4]] + [dev[4]]
    second = [x[:, 192:].contiguous() for x in dev[:4]] + [dev[4]]
    ya, sa = op(*first, return_state=True)
    yb, sb = op(*second, return_state=True, init_state=sa)
    torch.cuda.synchronize()
    y_ref, s_ref = oracle.forward_c(*ref, N)
    check_close("y", torch.cat([ya, yb], 1), y_ref, BF16)
    check_close("sT", sb, s_ref, BF16)


# The output stage (group norm over a head's channels, scale, offset, gate) fused into the block-form forward.
# (B, T, H, state): one pair per workgroup, a ragged end, several pairs per workgroup, one visit per pair
@pytest.mark.parametrize("B,T,H,with_state", [(5, 256, 32, True), (5, 250, 32, False), (40, 128, 32, True), (300, 64, 1, False),
                                              (13, 100, 40, True)])
def test_block_form_fused_output_stage(op, oracle, B, T, H, with_state):
    assert _pairs_in_range(B, H) or _several_pairs_per_workgroup(B, H)
    ins = oracle.make_inputs(B, T, H, N, 170 + T, with_state=True)
    if T >= 128:
        ins[3][B - 1, 40:60, 0:64] = 6.0     # one pair is redone exactly and then normalised in place
    dev, ref = cast_inputs(ins[:5], BF16)
    g = torch.Generator().manual_seed(T)
    gate_dev, gate_ref = cast_inputs([torch.randn(B, T, H * N, generator=g)], BF16)
    scale = torch.rand(H, N, generator=g) + 0.5
    offset = torch.randn(H, N, generator=g) * 0.3
    s0 = ins[6].float() if with_state else None
    op.algo = CHUNK
    out, sT = op.forward_gn_gate(*dev, gate_dev[0], scale.cuda(), offset.cuda(), 64e-5, return_state=True,
                                 init_state=s0.cuda() if with_state else None)
    torch.cuda.synchronize()
    y_ref, sT_ref = oracle.forward_c(*ref, N, to_np(s0) if with_state else None)
    want = oracle.group_norm_gate_np(y_ref, gate_ref[0], scale.numpy(), offset.numpy(), N, 64e-5)
    # (the norm divides by a head's standard deviation and so magnifies y's own rounding where that is small:
    # the stage's output is held to the composite bound, 1e-2 in the l2 norm and 3e-2 element-wise)
    check_composite("out", out, want)
    check_close("sT", sT, sT_ref, BF16)


# Gradients through the state (initial state in, gradient arriving at the final state, dL/dS_0 out) with one pair
# per workgroup: both given, either one, a ragged end, a pair redone exactly
@pytest.mark.parametrize("B,T,H,with_s0,with_gs,wild", [(5, 192, 32, True, True, False), (3, 128, 64, False, True, False),
                                                        (5, 100, 32, True, False, False), (129, 64, 1, True, True, False),
                                                        (5, 256, 32, True, True, True)])
def test_block_form_state_gradients(op, oracle, B, T, H, with_s0, with_gs, wild):
    from test_gpu_parity import _state_grad_case
    assert _pairs_in_range(B, H)
    _state_grad_case(op, oracle, B, T, H, 300 + T + H, BF16, CHUNK, with_s0=with_s0, with_gs=with_gs, wild=wild)


def test_either_forward_feeds_either_backward(oracle):
    """The saved chunk states have one layout: the block-form backward on the states of the fused (tile-form)
    forward -- what a training layer runs -- and the plain backward, which rebuilds the states with the
    tile form's state-only pass, agree with the saved pair to rounding and with the oracle."""
    from rwkv_kernel import _native

    lib = _native.load()
    B, T, H = 5, 256, 32
    C = H * N
    assert _pairs_in_range(B, H)
    ins = oracle.make_inputs(B, T, H, N, 88)
    dev, ref = cast_inputs(ins[:6], BF16)
    r, k, v, w, u, gy = dev
    st = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()
    n = lib.wkv6_saved_bytes(_native.BF16, CHUNK, B, T, C, H)
    g = torch.Generator().manual_seed(3)
    gate = torch.randn(B, T, C, generator=g).to(BF16).cuda()
    scale, offset = torch.ones(C, device="cuda"), torch.zeros(C, device="cuda")
    results = {}
    for mode in ("saved", "plain", "fused forward"):
        y = torch.empty_like(r)
        outs = [torch.full_like(r, float("nan")) for _ in range(4)] + [torch.empty(B, C, dtype=BF16, device="cuda")]
        buf = torch.empty(n, dtype=torch.uint8, device="cuda")
        if mode == "saved":
            _native.check(lib.wkv6_forward_save(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), P(buf), n))
        elif mode == "fused forward":
            out = torch.empty_like(r)
            stats = torch.empty(B, T, H, 2, device="cuda")
            _native.check(lib.wkv6_forward_gn_gate_save(st, _native.BF16, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gate), P(scale),
                                                        P(offset), 64e-5, P(out), P(y), P(stats), P(buf), n))
        if mode == "plain":
            _native.check(lib.wkv6_forward_ex(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(y), None, 0))
            _native.check(lib.wkv6_backward_ex(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                               *[P(o) for o in outs], P(buf), n))
        else:
            _native.check(lib.wkv6_backward_saved(st, _native.BF16, CHUNK, B, T, C, H, P(r), P(k), P(v), P(w), P(u), P(gy),
                                                  *[P(o) for o in outs], P(buf), n))
        torch.cuda.synchronize()
        results[mode] = [y] + outs
    y_ref, _ = oracle.forward_c(*ref[:5], N)
    g_ref = oracle.backward_c(*ref[:5], ref[5], N)
    for mode, (y, gr, gk, gv, gw, gu) in results.items():
        check_close(mode + " y", y, y_ref, BF16)
        for name, got, want in zip("gr gk gv gw".split(), (gr, gk, gv, gw), g_ref[:4]):
            check_close(mode + " " + name, got, want, BF16, is_grad=True)
        check_close(mode + " gu", to_np(gu).sum(0).reshape(H, N), g_ref[4], BF16, is_grad=True)
    for a, b in zip(results["saved"][1:5], results["fused forward"][1:5]):
        assert float((a.float() - b.float()).abs().max()) <= 2e-2 * float(a.float().abs().max())


def test_sequence_end_does_not_reach_back(oracle):
    """The first T tokens of a sequence that is 8 tokens longer (its last chunk then has tokens past the end,
    which are prepared as r = k = 0 with decay 1) give the y of the T-token sequence: bit for bit where the extra
    tokens have a chunk of their own, to rounding where they share the last chunk."""
    import rwkv_kernel

    op = rwkv_kernel.RWKVKernelOperator(N, 4096)
    B, H = 8, 32
    for T in (1024, 1000, 64):
        ins = oracle.make_inputs(B, T, H, N, 5)
        dev, _ = cast_inputs(ins[:5], BF16)
        op.algo = CHUNK
        with torch.no_grad():
            y1, s1 = op(*dev, return_state=True)
            longer = [torch.cat([x, x[:, :8]], 1).contiguous() for x in dev[:4]] + [dev[4]]
            y2, _ = op(*longer)
        torch.cuda.synchronize()
        if T % 64 == 0:
            assert torch.equal(y1, y2[:, :T]), T
        else:   # (the extra tokens share the last chunk: its blocks are scaled from other reference values)
            assert float((y1.float() - y2[:, :T].float()).abs().max()) <= 2e-2 * float(y1.float().abs().max()), T


# (B, T, H): sequence lengths that are no multiple of 64 -- one token more than a chunk, one less, T < 64, an odd
# number of chunks, several pairs per workgroup
@pytest.mark.parametrize("B,T,H", [(5, 250, 32), (3, 65, 64), (5, 63, 32), (129, 1, 1), (8, 1000, 32), (40, 100, 32), (75, 150, 4),
                                   (300, 33, 1)])
def test_block_form_ragged_sequence_end(op, oracle, B, T, H):
    assert _pairs_in_range(B, H) or _several_pairs_per_workgroup(B, H)
    print("block form, ragged B=%d T=%d H=%d" % (B, T, H), flush=True)
    y, grads, ref, gy_ref = _fwd_bwd(op, oracle.make_inputs(B, T, H, N, 800 + T + H))
    _check(oracle, y, grads, ref, gy_ref)
