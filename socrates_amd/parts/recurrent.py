"""Mixers that carry a state of fixed size per request instead of keys and values.

``WkvMixer``: time mixing with a matrix state per head and a decay per key channel that
depends on the token. ``Mamba2Mixer``: a state-space mixer with a scalar decay per head, a
short causal convolution in front and a gated group norm behind. Both keep their state (and
the few inputs of earlier tokens they still need) in one float32 tensor per cache slot,
``[rows, length]``, which the cache manager clears when a row opens; the kernels walk the
tokens of each sequence of the step in order, from the device's own copy of the sequence
starts, so a step may bring any portion of a prompt, and steps can be captured.
"""

from __future__ import annotations

import torch

from ..config.specs import Mamba2Spec, WkvSpec
from .registry import RowState, TensorDecl, register_part

_STREAMS = "rkvgw"       # the five blends of a token's input with the one before it


class WkvMixer:
    @staticmethod
    def tensors(spec: WkvSpec):
        d, C = spec.hidden, spec.n_heads * spec.head_dim
        rank = spec.decay_rank or -1
        t = {f"mu.{s}": TensorDecl((d,), "vector") for s in _STREAMS}
        t.update({s: TensorDecl((C, d)) for s in "rkvg"})
        t.update({"w1": TensorDecl((rank, d)), "w2": TensorDecl((C, rank)), "w0": TensorDecl((C,), "vector"),
                  "u": TensorDecl((spec.n_heads, spec.head_dim), "vector"), "norm": TensorDecl((C,), "vector"),
                  "o": TensorDecl((d, C))})
        return t

    @staticmethod
    def cache_need(spec: WkvSpec):
        # [the last token's input | the state, heads x key channels x value channels]
        return RowState((spec.hidden + spec.n_heads * spec.head_dim * spec.head_dim,))

    def __init__(self, spec: WkvSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.mu = torch.stack([tensors[f"mu.{s}"] for s in _STREAMS]).contiguous()
        self.w = {s: tensors[s] for s in "rkvgo"}
        self.w1, self.w0 = tensors["w1"], tensors["w0"]
        if self.w1.shape[0] != tensors["w2"].shape[1]:
            raise ValueError(f"wkv: the decay's two matrices do not fit ({tuple(self.w1.shape)}, {tuple(tensors['w2'].shape)})")
        self.w2_t = tensors["w2"].t().contiguous()          # [rank, channels]: the kernel's threads are channels
        self.bonus, self.gain = tensors["u"], tensors["norm"]

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        mixes = ops.token_shift(x, self.mu, slot.state, 0, ctx)
        r, k, v, g = (ops.linear(mixes[i], self.w[name]) for i, name in enumerate("rkvg"))
        decay = ops.wkv_decay(ops.linear(mixes[4], self.w1, out_dtype=torch.float32), self.w2_t, self.w0)
        o = ops.wkv(r, k, v, decay, g, self.bonus, self.gain, s.eps, s.n_heads, slot.state, s.hidden, ctx)
        return ops.linear(o, self.w["o"])


class Mamba2Mixer:
    @staticmethod
    def tensors(spec: Mamba2Spec):
        d, H, inner, C = spec.hidden, spec.n_heads, spec.inner, spec.conv_channels
        return {"in": TensorDecl((inner + C + H, d)),
                "conv": TensorDecl((C, spec.conv_taps), "vector"), "conv.b": TensorDecl((C,), "vector"),
                "dt_bias": TensorDecl((H,), "vector"), "A_log": TensorDecl((H,), "vector"),
                "D": TensorDecl((H,), "vector"), "norm": TensorDecl((inner,), "vector"),
                "o": TensorDecl((d, inner))}

    @staticmethod
    def cache_need(spec: Mamba2Spec):
        # [the convolution's last taps - 1 inputs, by tap and channel | the state, heads x state x head size]
        return RowState(((spec.conv_taps - 1) * spec.conv_channels + spec.n_heads * spec.state * spec.head_dim,))

    def __init__(self, spec: Mamba2Spec, tensors, ops):
        self.spec, self.ops = spec, ops
        w_in = tensors["in"]
        n = spec.inner + spec.conv_channels
        # step sizes enter the recurrence: their rows of the projection give float32 sums
        self.w_main, self.w_dt = w_in[:n].contiguous(), w_in[n:].contiguous()
        self.conv, self.conv_bias = tensors["conv"], tensors["conv.b"]
        self.dt_bias, self.a_log, self.skip = tensors["dt_bias"], tensors["A_log"], tensors["D"]
        self.gain, self.w_o = tensors["norm"], tensors["o"]
        self.adopted = 0

    def adopt(self, w):
        """Take ``w`` [n, hidden] as further rows of the input projection; ``forward`` then returns
        (y, x w^T). Returns the rows as they now lie (a view), for whoever held ``w``."""
        n = self.w_main.shape[0]
        self.w_main = torch.cat([self.w_main, w], dim=0).contiguous()
        self.adopted = w.shape[0]
        return self.w_main[n:]

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        zxbc = ops.linear(x, self.w_main)                                  # [N, z | x B C (| what was adopted)]
        dt = ops.linear(x, self.w_dt, out_dtype=torch.float32)
        xbc = ops.causal_conv_silu(zxbc, s.inner, s.conv_channels, self.conv, self.conv_bias, slot.state, 0, ctx)
        y = ops.ssd(xbc, dt, self.dt_bias, self.a_log, self.skip, s.n_heads, s.head_dim, s.state, s.n_groups,
                    slot.state, (s.conv_taps - 1) * s.conv_channels, ctx)
        y = ops.linear(ops.gated_group_norm(y, zxbc, self.gain, s.norm_groups, s.eps), self.w_o)
        return (y, zxbc[:, s.inner + s.conv_channels:]) if self.adopted else y


register_part(WkvSpec, WkvMixer)
register_part(Mamba2Spec, Mamba2Mixer)
