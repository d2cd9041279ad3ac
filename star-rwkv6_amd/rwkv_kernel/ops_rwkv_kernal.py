"""Portable python-loop flavour of the WKV6 operator (any device torch supports).

Mirrors the behaviour of the reference's backend-neutral operator
(rwkv_kernel/ops_rwkv_kernal.py:28-98): arithmetic in the input dtype, state argument handling,
and it ALWAYS returns (y, state).  Written on plain torch instead of keras.ops/bert4keras3.
It is selected only explicitly (KERAS_BACKEND neither "torch" nor "jax", or OPSKernelOperator);
the accelerated flavours never route through it.
"""
import torch


def _to_tensor(x):
    return x if isinstance(x, torch.Tensor) else getattr(x, "value", x)


class RWKVKernelOperator:
    def __init__(self, head_size, max_sequence_length):
        self.head_size = head_size
        self.max_sequence_length = max_sequence_length

    def __call__(self, r, k, v, w, u, with_state=False, init_state=None, state_map=None, return_state=None):
        # the reference spells the flag `with_state` here and `return_state` in the other flavours;
        # both are accepted and neither changes the result: (y, state) is always returned.
        N = self.head_size
        u = _to_tensor(u)
        B, T, C = r.shape
        assert C % N == 0
        H = C // N
        if init_state is not None:
            assert init_state.dim() in (3, 4), "init_state must be (state_kinds, H, N, N) or (H, N, N)"
            if init_state.dim() == 3:
                assert tuple(init_state.shape) == (H, N, N), "init_state must be (H, N, N)"
                init_state = init_state[None]
            else:
                assert tuple(init_state.shape[1:]) == (H, N, N), "init_state must be (state_kinds, H, N, N)"
                assert init_state.shape[0] <= B, "state_kinds must not exceed the batch size"
            kinds = init_state.shape[0]
            if state_map is None:
                if kinds == 1:
                    state_map = torch.zeros(B, dtype=torch.int64)
                elif kinds == B:
                    state_map = torch.arange(B, dtype=torch.int64)
                else:
                    raise ValueError("state_map cannot be inferred from init_state; pass it explicitly")
            else:
                if isinstance(state_map, (list, tuple)):
                    state_map = torch.tensor(state_map, dtype=torch.int64)
                assert state_map.dtype in (torch.int32, torch.int64), "state_map must be an integer array"
                state_map = state_map.to(torch.int64)
                assert bool((state_map >= 0).all()) and bool((state_map < kinds).all()), \
                    "state_map values must lie in [0, %d)" % kinds
            s = init_state.index_select(0, state_map.to(init_state.device))
        else:
            assert state_map is None
            s = torch.zeros(1, H, N, N, dtype=u.dtype, device=r.device)

        decay = torch.exp(-torch.exp(w.reshape(B, T, H, N, 1)))
        kc = k.reshape(B, T, H, N, 1)
        vr = v.reshape(B, T, H, 1, N)
        rr = r.reshape(B, T, H, 1, N)
        bonus = u.reshape(1, H, N, 1)
        outs = []
        for t in range(T):
            kv = kc[:, t] @ vr[:, t]
            outs.append((rr[:, t] @ (bonus * kv + s)).reshape(B, C))
            s = kv + decay[:, t] * s
        return torch.stack(outs, dim=1), s
