"""Retention: linear attention with a fixed decay per head and a matrix state per head and request.

One product reads the layer's input: rows [gate | q | k | v]. The recurrence kernel turns q and k by
position and scales k while it stages a batch of tokens, in float32, walks each sequence's tokens of
the step from the row's state (float32, zero when the row opens) and leaves the state for the next
step; a head's result is divided by its root mean square and multiplied by silu(gate) in the kernel
that serves the other recurrent mixers' head norms.
"""

from __future__ import annotations

import torch

from ..config.specs import RetentionSpec
from .gated_attention import rotation_frequencies
from .registry import RowState, TensorDecl, register_part


class RetentionMixer:
    @staticmethod
    def tensors(spec: RetentionSpec):
        H, D, Dv, d = spec.n_heads, spec.head_dim, spec.v_dim, spec.hidden
        return {"q": TensorDecl((H * D, d)), "k": TensorDecl((H * D, d)), "v": TensorDecl((H * Dv, d)),
                "g": TensorDecl((H * Dv, d)), "o": TensorDecl((d, H * Dv))}

    @staticmethod
    def cache_need(spec: RetentionSpec):
        return RowState((spec.n_heads * spec.head_dim * spec.v_dim,))

    def __init__(self, spec: RetentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, D, Dv = spec.n_heads, spec.head_dim, spec.v_dim
        self.w_first = torch.cat([tensors["g"], tensors["q"], tensors["k"], tensors["v"]], dim=0).contiguous()
        self.cols = (H * Dv, H * Dv + H * D, H * Dv + 2 * H * D)
        self.w_o = tensors["o"]
        self.decays = torch.tensor(spec.decays, dtype=torch.float64).to(torch.float32).to(ops.device)
        self.ones = torch.ones(H * Dv, dtype=torch.float32, device=ops.device)
        self.inv_freq, self.rotary_dim = rotation_frequencies(spec.position, ops.device)

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        first = ops.linear(x, self.w_first)
        raw = ops.retention(first, self.cols, s.n_heads, s.head_dim, s.v_dim, self.inv_freq, self.rotary_dim,
                            float(s.head_dim) ** -0.5, self.decays, slot.state, 0, ctx)
        o = ops.gated_group_norm(raw, first, self.ones, s.n_heads, s.eps, gate_first=False)
        return ops.linear(o, self.w_o)


register_part(RetentionSpec, RetentionMixer)
