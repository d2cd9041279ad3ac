"""rwkv_kernel: the WKV6 operator behind the package surface of infiy-quine/STAR-RWKV6.

    from rwkv_kernel import RWKVKernelOperator, OPSKernelOperator
    op = RWKVKernelOperator(head_size, max_sequence_length)
    y, state = op(r, k, v, w, u, return_state=False, init_state=None, state_map=None)

The flavour is picked by the KERAS_BACKEND environment variable, which must be set, exactly as
the reference does (rwkv_kernel/__init__.py:2-11): "torch" -> torch autograd.Function over the
gfx950 library, "jax" -> jax custom_vjp over the same library's XLA custom-call targets, anything
else -> the portable python-loop operator, which is also always exported as OPSKernelOperator.

State arguments (reference doc, rwkv_kernel/__init__.py:14-38):
  return_state  also return the final state; needed to pass init_state.
  init_state    (state_kinds, H, N, N) or (H, N, N), state_kinds <= batch; zero state if omitted.
                Indexed [key][value].  dtype: float32 when r is float16, else the dtype of r
                (float32 is additionally accepted for bfloat16 r, and then returned as float32).
  state_map     (batch,) int32/int64 tensor or list: batch row b starts from init_state[state_map[b]];
                values in [0, state_kinds).  Defaults: all zeros if state_kinds == 1, arange(batch) if
                state_kinds == batch, otherwise it must be given.
Returns (y, final_state or None).
"""
import os

assert "KERAS_BACKEND" in os.environ, "set KERAS_BACKEND to 'torch', 'jax' or another value for the python-loop flavour"

if os.environ["KERAS_BACKEND"] == "jax":
    from .jax_rwkv_kernel import RWKVKernelOperator
elif os.environ["KERAS_BACKEND"] == "torch":
    from .torch_rwkv_kernel import RWKVKernelOperator
else:
    from .ops_rwkv_kernal import RWKVKernelOperator

from .ops_rwkv_kernal import RWKVKernelOperator as OPSKernelOperator

__all__ = ["RWKVKernelOperator", "OPSKernelOperator"]
