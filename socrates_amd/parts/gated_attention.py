"""Grouped-query attention whose keys and values may differ in size, over a window that keeps the
first tokens visible, with one more weight of score 0 in the softmax's sum, values that may be
blended with an earlier layer's, and a gate per head.

One product reads the layer's input: rows [q | k | v | gate]. One kernel norms and turns q and k per
head, blends the values and writes keys and values to the token's place in the pages; both pools
have heads of ``cache_width`` elements (the larger of the two sizes, padded with zeros, which change
neither scores nor sums), so the paged-attention kernels that serve the other attention layers
serve this one, with the kept first keys and the added weight as further terms of theirs.
"""

from __future__ import annotations

import torch

from ..config.specs import GatedWindowAttentionSpec
from .registry import PagedKV, TensorDecl, register_part

_CARRY = "values of the first blended layer"


def rotation_frequencies(position, device):
    """float32 [rotary_dim / 2]: theta^(-2i / rotary_dim) / factor, evaluated in double precision."""
    if position is None:
        return None, 0
    dims = position.rotary_dim
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (position.theta ** (-2.0 * i / dims) / position.factor).to(torch.float32).to(device), dims


class GatedWindowAttention:
    @staticmethod
    def tensors(spec: GatedWindowAttentionSpec):
        H, G, D, Dv, d = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim, spec.hidden
        t = {"q": TensorDecl((H * D, d)), "k": TensorDecl((G * D, d)), "v": TensorDecl((G * Dv, d)),
             "o": TensorDecl((d, H * Dv))}
        if spec.qk_norm_eps is not None:
            t["q.norm"] = TensorDecl((D,), "vector")
            t["k.norm"] = TensorDecl((D,), "vector")
        if spec.value_blend is not None or spec.stores_blend:
            t["vmix"] = TensorDecl((), "vector")
        if spec.head_gate:
            t["g"] = TensorDecl((H, d))
        return t

    @staticmethod
    def cache_need(spec: GatedWindowAttentionSpec):
        return PagedKV(spec.n_kv_heads, spec.cache_width, spec.window, spec.keep_first if spec.window is not None else 0)

    def __init__(self, spec: GatedWindowAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, G, D, Dv = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim
        rows = [tensors["q"], tensors["k"], tensors["v"]] + ([tensors["g"]] if spec.head_gate else [])
        self.w_first = torch.cat(rows, dim=0).contiguous()
        self.w_q = self.w_first[:H * D]                     # all a layer needs that reads another's cache
        self.cols = (0, H * D, H * D + G * D)
        self.col_gate = H * D + G * D + G * Dv
        self.w_o = tensors["o"]
        self.q_gain, self.k_gain = tensors.get("q.norm"), tensors.get("k.norm")
        self.eps = spec.qk_norm_eps or 0.0
        self.lam = tensors["vmix"].to(torch.float32).reshape(1).contiguous() if spec.value_blend == "later" else None
        self.inv_freq, self.rotary_dim = rotation_frequencies(spec.position, ops.device)
        terms = {}
        if spec.sink:
            terms["sinks"] = torch.zeros(H, dtype=torch.float32, device=ops.device)
            terms["zero_sink"] = True            # (all of them zero: said here, so that nobody has to look)
        if spec.window is not None and spec.keep_first:
            terms["keep_first"] = spec.keep_first
        self.terms = terms or None

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        H, G, D, Dv, P = s.n_heads, s.n_kv_heads, s.head_dim, s.v_dim, s.cache_width
        if not write and s.head_gate:
            raise ValueError("a layer that reads another layer's cache has no gate of its own product here")
        first = ops.linear(x, self.w_first if write else self.w_q)
        earlier = None
        if write and s.value_blend == "first":
            ctx.carry[_CARRY] = first[:, self.cols[2]:self.cols[2] + G * Dv]
        elif write and s.value_blend == "later":
            earlier = ctx.carry[_CARRY]
        q = ops.attn_prepare(first, self.cols, H, G if write else 0, D, Dv, P, self.q_gain, self.k_gain, self.eps,
                             self.inv_freq, self.rotary_dim, ctx.positions, ctx.token_rows, slot if write else None,
                             earlier, self.lam if earlier is not None else None)
        o = ops.paged_attention(q, slot, ctx, s.scale, s.window, terms=self.terms)
        if s.head_gate or P != Dv:
            gate = first[:, self.col_gate:self.col_gate + H] if s.head_gate else None
            o = ops.head_gate(o, H, P, Dv, gate)
        return ops.linear(o, self.w_o)


register_part(GatedWindowAttentionSpec, GatedWindowAttention)
