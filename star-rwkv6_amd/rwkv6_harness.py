"""RWKV-6 model harness in plain torch around the WKV6 operator.

Measurement and test harness only: it exists so that the operator can be exercised the way its
caller does it -- once per layer, forward and backward, inside a real next-token training step --
without the Keras / bert4keras3 stack the reference's model file needs.  The layers restate
rwkv6_model.py of the reference, module by module:

    TimeShift        rwkv6_model.py:37-45    (x shifted right by one token) - x
    DecomposerDense  rwkv6_model.py:11-34    Dense(tanh, no bias) -> Dense(bias): the low-rank mixers
    TimeMix          rwkv6_model.py:117-185  data-dependent token-shift mixing, r/k/v/w/g projections,
                                             x, _ = rwkv_kernel(r, k, v, w, time_faaaa), per-head group
                                             norm (eps 64e-5), output projection of x * g
    ChannelMix       rwkv6_model.py:50-82    relu^2 key, sigmoid receptance
    GroupNorm        rwkv6_model.py:83-115
    Block            rwkv6_model.py:187-208  x + TimeMix(LN(x)); x + ChannelMix(LN(x))
    RWKV6            rwkv6_model.py:259-274  Embedding -> LN -> blocks -> LN -> Dense(vocab)

`rwkv_kernel` is any object with the operator's call signature `x, state = op(r, k, v, w, u)`:
rwkv_kernel.RWKVKernelOperator (the HIP library) on a GPU, rwkv_kernel.OPSKernelOperator (the
python loop) anywhere.  Initialisation is random (small normal / uniform decay range); no
checkpoint format is read or written here.
"""
import math

import torch
from torch import nn
import torch.nn.functional as F


def time_shift(x):
    """rwkv6_model.py:40-43: previous token (zero for the first) minus the token itself."""
    return F.pad(x, (0, 0, 1, 0))[:, :-1, :] - x


class DecomposerDense(nn.Module):
    def __init__(self, hidden_size, decomposer_size, use_bias=False):
        super().__init__()
        self.dense_a = nn.Linear(hidden_size, decomposer_size, bias=False)
        self.dense_b = nn.Linear(decomposer_size, hidden_size, bias=use_bias)

    def forward(self, x):
        return self.dense_b(torch.tanh(self.dense_a(x)))


class GroupNorm(nn.Module):
    """Layer norm over each head's channels with a per-(head, channel) scale and offset."""

    def __init__(self, hidden_size, head_size, epsilon=64e-5):
        super().__init__()
        assert hidden_size % head_size == 0
        self.num_heads, self.head_size, self.epsilon = hidden_size // head_size, head_size, epsilon
        self.scale = nn.Parameter(torch.ones(self.num_heads, head_size))
        self.offset = nn.Parameter(torch.zeros(self.num_heads, head_size))

    def forward(self, x):
        B, T, C = x.shape
        x = x.reshape(B, T, self.num_heads, self.head_size)
        x = F.layer_norm(x.float(), (self.head_size,), None, None, self.epsilon).to(x.dtype)
        return (self.scale.to(x.dtype) * x + self.offset.to(x.dtype)).reshape(B, T, C)


class TimeMix(nn.Module):
    def __init__(self, rwkv_kernel, hidden_size, decomposer_size, head_size):
        super().__init__()
        assert hidden_size % head_size == 0
        self.rwkv_kernel = rwkv_kernel
        self.hidden_size, self.head_size = hidden_size, head_size
        self.time_mix_x = nn.Parameter(torch.rand(hidden_size))
        self.dense_xr = DecomposerDense(hidden_size, decomposer_size, use_bias=True)
        self.dense_xw = DecomposerDense(hidden_size, decomposer_size, use_bias=True)
        self.dense_xk = DecomposerDense(hidden_size, decomposer_size, use_bias=True)
        self.dense_xv = DecomposerDense(hidden_size, decomposer_size, use_bias=True)
        self.dense_xg = DecomposerDense(hidden_size, decomposer_size, use_bias=True)
        self.dense_r = nn.Linear(hidden_size, hidden_size, bias=False)
        self.dense_k = nn.Linear(hidden_size, hidden_size, bias=False)
        self.dense_v = nn.Linear(hidden_size, hidden_size, bias=False)
        self.dense_w = DecomposerDense(hidden_size, head_size, use_bias=True)
        self.dense_g = nn.Linear(hidden_size, hidden_size, bias=False)
        self.time_faaaa = nn.Parameter(0.5 * torch.randn(hidden_size // head_size, head_size))
        self.group_norm = GroupNorm(hidden_size, head_size)
        self.dense_o = nn.Linear(hidden_size, hidden_size, bias=False)
        # the raw decay input w: the bias spreads it over [-6, 1] (decay exp(-exp(w)) from 0.998 to 0.07)
        with torch.no_grad():
            self.dense_w.dense_b.bias.uniform_(-6.0, 1.0)

    def _mixed_inputs(self, x):
        """xr, xk, xv, xw, xg of rwkv6_model.py:134-145."""
        mixers = (self.dense_xr, self.dense_xk, self.dense_xv, self.dense_xw, self.dense_xg)
        fused = getattr(self.rwkv_kernel, "shift_mix", None)
        if fused is not None and x.is_cuda and torch.is_autocast_enabled('cuda') and torch.get_autocast_dtype('cuda') == torch.bfloat16:
            xb = x.to(torch.bfloat16).contiguous()
            if self.rwkv_kernel.shift_mix_supported(xb, mixers[0].dense_a.out_features):
                # token shift, x_mix and the five rank-R expansions in the operator library's kernels
                return fused(xb, self.time_mix_x,
                             torch.cat([m.dense_a.weight for m in mixers]),
                             torch.stack([m.dense_b.weight for m in mixers]),
                             torch.stack([m.dense_b.bias for m in mixers]))
        x_shift = time_shift(x)
        x_mix = x + x_shift * self.time_mix_x.to(x.dtype)
        return tuple(x + x_shift * m(x_mix) for m in mixers)

    def forward(self, x, mask=None):
        xr, xk, xv, xw, xg = self._mixed_inputs(x)
        r, k, v, w, g = self.dense_r(xr), self.dense_k(xk), self.dense_v(xv), self.dense_w(xw), F.silu(self.dense_g(xg))
        if mask is not None:
            # Padded tokens neither write to the state nor decay it.  rwkv6_model.py:149-152 sets
            # w = -1e9 there (decay 1) and multiplies xk by the mask -- after k has already been
            # computed from xk (:148), so in the reference as committed k stays unmasked and a padded
            # token still writes k v^T into the state.  The evident intent is implemented here: k is
            # masked.  (A deliberate deviation; the operator itself is not involved.)
            m = mask.to(x.dtype)[..., None]
            k = k * m
            w = w * m + (1 - m) * -1e9
        u = self.time_faaaa.to(r.dtype)
        fused = getattr(self.rwkv_kernel, "forward_gn_gate", None)
        if fused is not None and r.is_cuda and r.dtype == torch.bfloat16:
            # group norm and gate come out of the operator's own output stage (inference: y is never
            # written; training: y and the norm's statistics are kept for one fused backward kernel)
            x, _ = fused(r.contiguous(), k.contiguous(), v.contiguous(), w.contiguous(), u, g.contiguous(),
                         self.group_norm.scale, self.group_norm.offset, self.group_norm.epsilon)
            return self.dense_o(x)
        y, _ = self.rwkv_kernel(r.contiguous(), k.contiguous(), v.contiguous(), w.contiguous(), u)
        return self.dense_o(self.group_norm(y) * g)


class ChannelMix(nn.Module):
    def __init__(self, hidden_size, expand_size, rwkv_kernel=None):
        super().__init__()
        self.rwkv_kernel = rwkv_kernel   # optional: its shift_mix_x kernel does the two token-shift mixes in bf16
        self.time_mix_k = nn.Parameter(torch.rand(hidden_size))
        self.time_mix_r = nn.Parameter(torch.rand(hidden_size))
        self.dense_key = nn.Linear(hidden_size, expand_size, bias=False)
        self.dense_value = nn.Linear(expand_size, hidden_size, bias=False)
        self.dense_receptance = nn.Linear(hidden_size, hidden_size, bias=False)

    def forward(self, x):
        fused = getattr(self.rwkv_kernel, "shift_mix_x", None)
        if fused is not None and x.is_cuda and torch.is_autocast_enabled('cuda') and torch.get_autocast_dtype('cuda') == torch.bfloat16 \
                and x.shape[-1] % 64 == 0:
            xb = x.to(torch.bfloat16).contiguous()
            xk, xr = fused(xb, self.time_mix_k), fused(xb, self.time_mix_r)
        else:
            xx = time_shift(x)
            xk = x + xx * self.time_mix_k.to(x.dtype)
            xr = x + xx * self.time_mix_r.to(x.dtype)
        k = torch.square(torch.relu(self.dense_key(xk)))
        return torch.sigmoid(self.dense_receptance(xr)) * self.dense_value(k)


class Block(nn.Module):
    def __init__(self, rwkv_kernel, hidden_size, decomposer_size, head_size, expand_size):
        super().__init__()
        self.layer_norm_att = nn.LayerNorm(hidden_size, eps=1e-5)
        self.layer_norm_ffn = nn.LayerNorm(hidden_size, eps=1e-5)
        self.time_mix = TimeMix(rwkv_kernel, hidden_size, decomposer_size, head_size)
        self.channel_mix = ChannelMix(hidden_size, expand_size, rwkv_kernel)

    def forward(self, x, mask=None):
        x = x + self.time_mix(self.layer_norm_att(x), mask)
        return x + self.channel_mix(self.layer_norm_ffn(x))


class RWKV6(nn.Module):
    def __init__(self, rwkv_kernel, num_layers, vocabulary_size, hidden_size, decomposer_size, head_size, expand_size):
        super().__init__()
        self.embedding = nn.Embedding(vocabulary_size, hidden_size)
        self.embedding_ln = nn.LayerNorm(hidden_size, eps=1e-5)
        self.blocks = nn.ModuleList(Block(rwkv_kernel, hidden_size, decomposer_size, head_size, expand_size)
                                    for _ in range(num_layers))
        self.output_ln = nn.LayerNorm(hidden_size, eps=1e-5)
        self.output_layer = nn.Linear(hidden_size, vocabulary_size, bias=False)
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, std=0.5 / math.sqrt(m.in_features))
        nn.init.normal_(self.embedding.weight, std=0.02)

    def forward(self, ids, mask=None):
        x = self.embedding_ln(self.embedding(ids))
        for blk in self.blocks:
            x = blk(x, mask)
        return self.output_layer(self.output_ln(x))


def train_step(model, optimizer, ids, autocast_dtype=None):
    """One next-token cross-entropy step: forward, backward, optimizer update.  Returns the loss."""
    optimizer.zero_grad(set_to_none=True)
    dev = ids.device.type
    with torch.autocast(dev, dtype=autocast_dtype, enabled=autocast_dtype is not None):
        logits = model(ids[:, :-1])
    loss = F.cross_entropy(logits.float().reshape(-1, logits.shape[-1]), ids[:, 1:].reshape(-1))
    loss.backward()
    optimizer.step()
    return loss.detach()


# the layer shape of configuration 4: RWKV6-1.6B (24 layers, d_model 2048, 32 heads of 64, FFN 7168)
CONFIG4 = dict(num_layers=24, vocabulary_size=65536, hidden_size=2048, decomposer_size=32, head_size=64, expand_size=7168)
