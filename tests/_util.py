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
