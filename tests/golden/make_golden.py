"""Writes tests/golden/wkv6_small.npz: seeded inputs and the expected outputs.

The reference stores no vectors for WKV6, and its python loop is fully pinned by closed forms
(tests/test_oracle.py), so the expected values here come from torch.autograd through the
float64 python-loop restatement (oracle.wkv6_ref.loop_torch), NOT from importing reference code.
The fixture guards the C oracle and the HIP kernels against regressions.
Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import wkv6_ref  # noqa: E402

B, T, H, N = 2, 16, 2, 64
r, k, v, w, u, gy, s0 = wkv6_ref.make_inputs(B, T, H, N, seed=1234, with_state=True)
smap = torch.tensor([1, 0])
d = [x.double() for x in (r, k, v, w, u)]
y, _ = wkv6_ref.loop_torch(*d, N)
ys, sT = wkv6_ref.loop_torch(*d, N, s0.double(), smap)
gr, gk, gv, gw, gu = wkv6_ref.grads_torch(*d, gy.double(), N)
np.savez_compressed(
    os.path.join(os.path.dirname(os.path.abspath(__file__)), "wkv6_small.npz"),
    head_size=N, r=r.numpy(), k=k.numpy(), v=v.numpy(), w=w.numpy(), u=u.numpy(), gy=gy.numpy(),
    s0=s0.numpy(), state_map=smap.numpy(), y=y.numpy(), y_state=ys.numpy(), sT=sT.numpy(),
    gr=gr.numpy(), gk=gk.numpy(), gv=gv.numpy(), gw=gw.numpy(), gu=gu.numpy())
print("written")
