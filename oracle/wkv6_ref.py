"""CPU oracle for the WKV6 operator.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module;
the shipped rwkv_kernel package never does.

Three independent restatements of the same operator (citations relative to the reference tree):

* ``loop_torch``      -- the python time loop of rwkv_kernel/ops_rwkv_kernal.py:28-98
                         (== rwkv_v6_demo.py:10-43) in plain torch; differentiable, so
                         torch.autograd through it is the gradient definition the reference
                         itself uses (deprecated_code/wkv_torch.py:56).
* ``closed_form_np``  -- the O(T^2) unrolled sum, numpy float64, for brute force on tiny shapes.
* ``forward_c`` / ``backward_c`` -- oracle/wkv6_oracle.c through ctypes (double or float), fast
                         enough for full benchmark shapes; gradients in adjoint form.

Conventions: r,k,v,w,y,gy : (B,T,C), c = h*N+n;  u : (H,N);  state : (B,H,N,N) indexed
[key j][value i] (rwkv_kernel/ops_rwkv_kernal.py:85-91);  w is the RAW decay input, the operator
applies exp(-exp(w)) itself (rwkv_kernel/jax_kernel/rwkv_kernels.cu:125).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwkv6_oracle.so")
_lib = None


def build_c_oracle(force=False):
    """Compile oracle/wkv6_oracle.c with the Makefile beside it."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build_c_oracle()
        _lib = ctypes.CDLL(_LIB_PATH)
        i64, p = ctypes.c_int64, ctypes.c_void_p
        for sfx in ("_f64", "_f32"):
            f = getattr(_lib, "wkv6_oracle_forward" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [i64] * 4 + [p] * 7 + [i64] + [p] * 2
            g = getattr(_lib, "wkv6_oracle_backward" + sfx)
            g.restype = ctypes.c_int
            g.argtypes = [i64] * 4 + [p] * 11
            gs = getattr(_lib, "wkv6_oracle_backward_state" + sfx)
            gs.restype = ctypes.c_int
            gs.argtypes = [i64] * 4 + [p] * 14
    return _lib


def _as(a, dt):
    return np.ascontiguousarray(np.asarray(a, dtype=dt))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def forward_c(r, k, v, w, u, head_size, init_state=None, state_map=None, dtype=np.float64):
    """y, final_state from the C oracle.  Arithmetic in ``dtype`` (float64 or float32)."""
    lib = _load()
    r, k, v, w = (_as(x, dtype) for x in (r, k, v, w))
    B, T, C = r.shape
    N = head_size
    H = C // N
    u = _as(u, dtype).reshape(H, N)
    s0 = m = None
    n_state = 0
    if init_state is not None:
        s0 = _as(init_state, dtype)
        if s0.ndim == 3:
            s0 = s0[None]
        n_state = s0.shape[0]
        if state_map is None:
            state_map = np.zeros(B, np.int64) if n_state == 1 else np.arange(B)
        m = _as(state_map, np.int64)
    y = np.empty((B, T, C), dtype)
    sT = np.empty((B, H, N, N), dtype)
    sfx = "_f64" if dtype == np.float64 else "_f32"
    rc = getattr(lib, "wkv6_oracle_forward" + sfx)(
        B, T, H, N, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(s0), _ptr(m), n_state, _ptr(y), _ptr(sT))
    if rc != 0:
        raise ValueError("state_map entry out of range")
    return y, sT


def backward_c(r, k, v, w, u, gy, head_size, dtype=np.float64):
    """gr, gk, gv, gw, gu(H,N) of the stateless operator from the C oracle (adjoint form)."""
    lib = _load()
    r, k, v, w, gy = (_as(x, dtype) for x in (r, k, v, w, gy))
    B, T, C = r.shape
    N = head_size
    H = C // N
    u = _as(u, dtype).reshape(H, N)
    gr, gk, gv, gw = (np.empty((B, T, C), dtype) for _ in range(4))
    gu = np.empty((B, C), dtype)
    sfx = "_f64" if dtype == np.float64 else "_f32"
    rc = getattr(lib, "wkv6_oracle_backward" + sfx)(
        B, T, H, N, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(gy),
        _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu))
    if rc != 0:
        raise MemoryError("oracle backward failed")
    return gr, gk, gv, gw, gu.sum(0).reshape(H, N)


def backward_state_c(r, k, v, w, u, gy, head_size, init_state=None, g_state=None, dtype=np.float64):
    """Gradients of  sum(y*gy) + sum(S_T*g_state)  with S_0 = init_state (B,H,N,N; None = 0):
    gr, gk, gv, gw, gu(H,N), gs0 (B,H,N,N) from the C oracle (adjoint form).  The operator the
    reference defines has no gradient through the state; this is the extension the carried-state
    API suggests (dL/dS_0 = G_0, G_T = g_state)."""
    lib = _load()
    r, k, v, w, gy = (_as(x, dtype) for x in (r, k, v, w, gy))
    B, T, C = r.shape
    N = head_size
    H = C // N
    u = _as(u, dtype).reshape(H, N)
    s0 = None if init_state is None else _as(init_state, dtype).reshape(B, H, N, N)
    gsT = None if g_state is None else _as(g_state, dtype).reshape(B, H, N, N)
    gr, gk, gv, gw = (np.empty((B, T, C), dtype) for _ in range(4))
    gu = np.empty((B, C), dtype)
    gs0 = np.empty((B, H, N, N), dtype)
    sfx = "_f64" if dtype == np.float64 else "_f32"
    rc = getattr(lib, "wkv6_oracle_backward_state" + sfx)(
        B, T, H, N, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(s0), _ptr(gy), _ptr(gsT),
        _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu), _ptr(gs0))
    if rc != 0:
        raise MemoryError("oracle backward failed")
    return gr, gk, gv, gw, gu.sum(0).reshape(H, N), gs0


def loop_torch(r, k, v, w, u, head_size, init_state=None, state_map=None):
    """The reference's python loop (rwkv_kernel/ops_rwkv_kernal.py:28-98) in torch.

    Arithmetic stays in the input dtype (the loop does no upcast, :74-93).  Returns (y, s)
    always, like the reference (:96-98).  Differentiable.
    """
    import torch

    B, T, C = r.shape
    N = head_size
    assert C % N == 0
    H = C // N
    w5 = w.reshape(B, T, H, N, 1)
    k5 = k.reshape(B, T, H, N, 1)
    v5 = v.reshape(B, T, H, 1, N)
    r5 = r.reshape(B, T, H, 1, N)
    u4 = u.reshape(1, H, N, 1)
    if init_state is not None:
        if init_state.dim() == 3:
            init_state = init_state[None]
        n_state = init_state.shape[0]
        if state_map is None:
            if n_state == 1:
                state_map = torch.zeros(B, dtype=torch.int64)
            elif n_state == B:
                state_map = torch.arange(B, dtype=torch.int64)
            else:
                raise ValueError("cannot infer state_map")
        state_map = torch.as_tensor(state_map, dtype=torch.int64)
        assert bool((state_map >= 0).all()) and bool((state_map < n_state).all())
        s = init_state.index_select(0, state_map.to(init_state.device))
    else:
        s = torch.zeros(1, H, N, N, dtype=u.dtype, device=u.device)
    d5 = torch.exp(-torch.exp(w5))
    ys = []
    for t in range(T):
        kv = k5[:, t] @ v5[:, t]
        ys.append((r5[:, t] @ (u4 * kv + s)).reshape(B, C))
        s = kv + d5[:, t] * s
    return torch.stack(ys, 1).reshape(B, T, C), s


def grads_torch(r, k, v, w, u, gy, head_size):
    """Gradients of sum(y*gy) wrt r,k,v,w,u by torch.autograd through ``loop_torch``."""
    import torch

    leaves = [x.detach().clone().requires_grad_(True) for x in (r, k, v, w, u)]
    y, _ = loop_torch(*leaves, head_size)
    return torch.autograd.grad(y, leaves, grad_outputs=gy)


def closed_form_np(r, k, v, w, u, head_size, init_state=None):
    """y by the unrolled O(T^2) sum (float64):
    y_t[i] = sum_j r_t[j] ( u_j k_t[j] v_t[i] + prod_{s<t} d_s[j] S0[j][i]
                            + sum_{tau<t} k_tau[j] v_tau[i] prod_{tau<s<t} d_s[j] ).
    init_state, if given, is (B,H,N,N).  Tiny shapes only."""
    r, k, v, w = (np.asarray(x, np.float64) for x in (r, k, v, w))
    B, T, C = r.shape
    N = head_size
    H = C // N
    u = np.asarray(u, np.float64).reshape(H, N)
    d = np.exp(-np.exp(w))
    y = np.zeros((B, T, C))
    for b in range(B):
        for h in range(H):
            sl = slice(h * N, (h + 1) * N)
            for t in range(T):
                acc = (r[b, t, sl] * u[h] * k[b, t, sl]).sum() * v[b, t, sl]
                for tau in range(t):
                    decay = np.prod(d[b, tau + 1:t, sl], axis=0)
                    acc = acc + (r[b, t, sl] * decay * k[b, tau, sl]).sum() * v[b, tau, sl]
                if init_state is not None:
                    decay0 = np.prod(d[b, 0:t, sl], axis=0)
                    acc = acc + (r[b, t, sl] * decay0) @ np.asarray(init_state, np.float64)[b, h]
                y[b, t, sl] = acc
    return y


def group_norm_gate_np(y, gate, scale, offset, head_size, epsilon=64e-5):
    """What the caller does with the operator's output in the reference model, in float64:
    per-head layer norm of y with scale and offset (rwkv6_model.py:94-99: mean and variance over
    one head's channels, 1/sqrt(var + epsilon)), then the gate (rwkv6_model.py:158-160)."""
    y = np.asarray(y, dtype=np.float64)
    B, T, C = y.shape
    N = head_size
    H = C // N
    x = y.reshape(B, T, H, N)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    x = (x - mu) / np.sqrt(var + epsilon)
    x = x * np.asarray(scale, dtype=np.float64).reshape(1, 1, H, N) + np.asarray(offset, dtype=np.float64).reshape(1, 1, H, N)
    return x.reshape(B, T, C) * np.asarray(gate, dtype=np.float64)


def shift_mix_np(x, mix_x, a, w2t, bias):
    """What the reference model does with the layer input before the projections that feed the
    operator, in float64 (rwkv6_model.py:134-146):
        xx = TimeShift(x) = (x padded with one zero token in front, last dropped) - x       :40-43
        x_mix = x + xx * mix_x                                                              :136
        coef_s = DecomposerDense_s(x_mix) = tanh(x_mix a_s^T) w2t_s^T + bias_s              :11-25, :139
        x_s = x + xx * coef_s  for s = r, k, v, w, g                                        :141-145
    a (5R, C): dense_a kernels stacked, as (out, in); w2t (5, C, R): dense_b kernels as (out, in);
    bias (5, C).  Returns (x_mix, h (B,T,5,R), [xr, xk, xv, xw, xg])."""
    x = np.asarray(x, dtype=np.float64)
    B, T, C = x.shape
    w2t = np.asarray(w2t, dtype=np.float64)
    R = w2t.shape[2]
    prev = np.concatenate([np.zeros((B, 1, C)), x[:, :-1]], axis=1)
    xx = prev - x
    x_mix = x + xx * np.asarray(mix_x, dtype=np.float64).reshape(1, 1, C)
    h = np.tanh(x_mix @ np.asarray(a, dtype=np.float64).T).reshape(B, T, 5, R)
    outs = []
    for s in range(5):
        coef = h[:, :, s, :] @ w2t[s].T + np.asarray(bias, dtype=np.float64)[s].reshape(1, 1, C)
        outs.append(x + xx * coef)
    return x_mix, h, outs


def make_inputs(B, T, H, N, seed, with_gy=True, with_state=False):
    """The benchmark's seeded distributions, drawn on the CPU in float32:
    r,k,v ~ N(0,1); w = x ~ U(-6,1) passed raw; u ~ N(0,0.5^2) (H,N); gy ~ N(0,1);
    h0 ~ N(0,0.1^2) (B,H,N,N)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    C = H * N
    r = torch.randn(B, T, C, generator=g)
    k = torch.randn(B, T, C, generator=g)
    v = torch.randn(B, T, C, generator=g)
    w = torch.rand(B, T, C, generator=g) * 7.0 - 6.0
    u = torch.randn(H, N, generator=g) * 0.5
    out = [r, k, v, w, u]
    if with_gy:
        out.append(torch.randn(B, T, C, generator=g))
    if with_state:
        out.append(torch.randn(B, H, N, N, generator=g) * 0.1)
    return out
