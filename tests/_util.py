"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

# Tolerances of the parity contract.
#   fp32 tensors : max|y - y_ref| <= 1e-4 ; gradients: max|g - g_ref| / max|g_ref| <= 1e-3
#   bf16 / fp16  : max|x - x_ref| / max|x_ref| <= 1e-2 and ||x - x_ref||_2 / ||x_ref||_2 <= 1e-2
# The reference values are always the float64 oracle fed the SAME (already rounded) inputs.
TOL_F32_Y_ABS = 1e-4
TOL_F32_GRAD_REL = 1e-3
TOL_LOWP_REL = 1e-2


def rel_inf(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def rel_l2(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.linalg.norm((got - ref).ravel()) / max(np.linalg.norm(ref.ravel()), 1e-30))


def to_np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def out_dtype(dt):
    return torch.float32 if dt == torch.float16 else dt


def cast_inputs(tensors, dtype, device="cuda"):
    """Round the seeded fp32 tensors to `dtype`; returns (device tensors, float64 numpy views of
    exactly those rounded values for the oracle)."""
    dev = [t.to(dtype).to(device).contiguous() for t in tensors]
    ref = [to_np(t) for t in dev]
    return dev, ref


def check_close(name, got, ref, dtype, is_grad=False):
    got = to_np(got) if isinstance(got, torch.Tensor) else got
    if dtype == torch.float32:
        if is_grad:
            e = rel_inf(got, ref)
            assert e <= TOL_F32_GRAD_REL, "%s: rel-inf %.3e > %.1e" % (name, e, TOL_F32_GRAD_REL)
        else:
            e = float(np.abs(got - ref).max())
            assert e <= TOL_F32_Y_ABS * max(1.0, np.abs(ref).max() / 64.0), "%s: max-abs %.3e" % (name, e)
    else:
        e1, e2 = rel_inf(got, ref), rel_l2(got, ref)
        assert e1 <= TOL_LOWP_REL and e2 <= TOL_LOWP_REL, "%s: rel-inf %.3e rel-l2 %.3e > %.1e" % (name, e1, e2, TOL_LOWP_REL)
    assert np.isfinite(got).all(), name + " has non-finite values"


def flat_heads(y_ref, N, frac=0.05):
    """(B, T, H) mask of the (token, head) groups whose standard deviation over the head's N channels is
    below `frac` of the median one.  There the per-head norm is ill-conditioned: 1/std magnifies the
    bf16 rounding of y itself into the gradient wrt y, whatever computes it.  With random inputs the
    first tokens of a sequence (y_0 is one scalar times v_0) produce a few such groups among many pairs."""
    B, T, C = y_ref.shape
    sd = y_ref.reshape(B, T, C // N, N).std(-1)
    return sd < frac * np.median(sd)


def fused_stage_reference(oracle, ref_inputs, gate_ref, gout_ref, scale, offset, N, eps, y_ref=None):
    """float64 values of the fused training stage out = (layer_norm(y) * scale + offset) * gate for the
    (already rounded) operator inputs `ref_inputs` = [r, k, v, w, u]: the oracle's y, torch's layer_norm
    autograd for the norm and the gate, the oracle's backward for the operator fed that stage's gradient
    wrt y rounded to bf16 (as the kernel hands it on).  Returns a dict of numpy arrays."""
    B, T, C = ref_inputs[0].shape
    H = C // N
    if y_ref is None:
        y_ref, _ = oracle.forward_c(*ref_inputs, N)
    yt = torch.tensor(y_ref, dtype=torch.float64, requires_grad=True)
    gt = torch.tensor(gate_ref, dtype=torch.float64, requires_grad=True)
    st = torch.tensor(np.asarray(scale, np.float64), requires_grad=True)
    ot = torch.tensor(np.asarray(offset, np.float64), requires_grad=True)
    z = torch.nn.functional.layer_norm(yt.view(B, T, H, N), (N,), eps=eps)
    out = (z * st + ot).view(B, T, C) * gt
    out.backward(torch.tensor(gout_ref, dtype=torch.float64))
    gy_ref = yt.grad.to(torch.bfloat16).double().numpy()
    want = dict(out=out.detach().numpy(), ggate=gt.grad.numpy(), gscale=st.grad.numpy(), goffset=ot.grad.numpy())
    want.update(zip("gr gk gv gw gu".split(), oracle.backward_c(*ref_inputs, gy_ref, N)))
    return want


def check_composite(name, got, want):
    """Tolerance of the fused training stage.  The norm divides by a head's standard deviation, which
    magnifies the operator's own error in y (within its 1e-2) where that deviation is small, and the
    operator's gradients sit behind two bf16 roundings (y, gy) and the norm's backward: the composite is
    held to 1e-2 in the l2 norm and 3e-2 element-wise."""
    got = to_np(got) if isinstance(got, torch.Tensor) else np.asarray(got, np.float64)
    got = got.reshape(want.shape)
    assert np.isfinite(got).all(), name
    e1, e2 = rel_inf(got, want), rel_l2(got, want)
    assert e2 <= 1e-2 and e1 <= 3e-2, "%s: rel-l2 %.3e rel-inf %.3e" % (name, e2, e1)
