"""Attention over one cached latent per token.

A token leaves [latent | rotated key part] in the cache; per head the plain key is Wuk latent
and the value Wuv latent. Neither is ever built: with q' = Wuk_h^T q_plain the plain score is
q' . latent, so a head's query becomes [q' | q_rot] against the cached vector itself, all
heads share that one "key head", the weighted sum of the cached vectors is taken by the same
paged-attention kernels that serve grouped-query layers (keys and values are the one pool),
and Wuv_h turns the latent part of the sum into the head's output. The cache holds
``cache_width`` elements per token and a window of them.
"""

from __future__ import annotations

import torch

from ..config.specs import LatentAttentionSpec
from .registry import PagedLatent, TensorDecl, register_part


class LatentAttention:
    @staticmethod
    def tensors(spec: LatentAttentionSpec):
        H, R = spec.n_heads, spec.kv_rank
        t = {"dq": TensorDecl((spec.q_rank, spec.hidden)), "dq.norm": TensorDecl((spec.q_rank,), "vector"),
             "uq": TensorDecl((H * (spec.head_dim + spec.rot_dim), spec.q_rank)),
             "uk": TensorDecl((H * spec.head_dim, R)), "uv": TensorDecl((H * spec.v_dim, R)),
             "o": TensorDecl((spec.hidden, H * spec.v_dim))}
        if spec.own_kv:
            t["dkv"] = TensorDecl((R + spec.rot_dim, spec.hidden))
            t["dkv.norm"] = TensorDecl((R,), "vector")
        return t

    @staticmethod
    def cache_need(spec: LatentAttentionSpec):
        return PagedLatent(spec.cache_width, spec.keep)

    def __init__(self, spec: LatentAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, D, R = spec.n_heads, spec.head_dim, spec.kv_rank
        self.q_gain, self.w_uq = tensors["dq.norm"], tensors["uq"]
        # one product for everything that reads the layer's input: rows [query latent | latent and key part]
        # (and, behind them, what the block has this part adopt)
        self.w_first = (torch.cat([tensors["dq"], tensors["dkv"]], dim=0).contiguous() if spec.own_kv else tensors["dq"])
        self.n_own = self.w_first.shape[0]
        self.adopted = 0
        # per head [R, D]: the product that folds a head's plain query into the latent's space
        self.w_uk_t = tensors["uk"].view(H, D, R).transpose(1, 2).contiguous()
        self.w_uv = tensors["uv"].view(H, spec.v_dim, R).contiguous()
        self.w_o = tensors["o"]
        self.kv_gain = tensors.get("dkv.norm")
        # pair i of the rotated part turns by position * base^(-2i / dims)
        dims = spec.position.dims
        i = torch.arange(dims // 2, dtype=torch.float64)
        self.inv_freq = (spec.position.base ** (-2.0 * i / dims)).to(torch.float32).to(ops.device)

    def adopt(self, w):
        """Take ``w`` [n, hidden] as further rows of the first product; ``forward`` then returns (y, x w^T).
        Returns the rows as they now lie (a view), for whoever held ``w``."""
        self.w_first = torch.cat([self.w_first, w], dim=0).contiguous()
        self.adopted = w.shape[0]
        return self.w_first[self.n_own:]

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        if write != s.own_kv:
            raise ValueError("a latent-attention layer writes the cache slot exactly if it has a down-projection of its own")
        first = ops.linear(x, self.w_first)
        q = ops.linear(ops.rmsnorm_cols(first[:, :s.q_rank], self.q_gain, s.eps), self.w_uq)
        if write:
            ops.latent_write(first[:, s.q_rank:s.q_rank + s.kv_rank + s.rot_dim], s.kv_rank, s.rot_dim, self.kv_gain, s.eps,
                             self.inv_freq, ctx.positions, ctx.token_rows, slot)
        folded = ops.latent_query(q, s.n_heads, s.head_dim, s.rot_dim, self.w_uk_t, s.cache_width, self.inv_freq,
                                  ctx.positions)
        mixed = ops.paged_attention(folded, slot, ctx, s.scale, s.window)
        o = ops.head_project(mixed.view(-1, s.n_heads, s.cache_width), self.w_uv)
        y = ops.linear(o, self.w_o)
        return (y, first[:, self.n_own:]) if self.adopted else y


register_part(LatentAttentionSpec, LatentAttention)
