"""A per-layer input that depends on the token alone: a few columns of a table that all layers
share, gated by the residual stream, projected to the width and RMS-normed into the stream."""

from __future__ import annotations

from ..config.specs import TokenSideSpec
from .registry import TensorDecl, register_part


class TokenSide:
    @staticmethod
    def tensors(spec: TokenSideSpec):
        # (a local name that starts with "/" is a name of the whole model: every layer reads the same tensor)
        return {"gate": TensorDecl((spec.dim, spec.hidden)), "proj": TensorDecl((spec.hidden, spec.dim)),
                "norm": TensorDecl((spec.hidden,), "vector"),
                "/" + spec.table_name: TensorDecl((spec.vocab, spec.n_layers * spec.dim))}

    def __init__(self, spec: TokenSideSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.w_gate, self.w_proj, self.gain = tensors["gate"], tensors["proj"], tensors["norm"]
        self.table = tensors["/" + spec.table_name]
        self.eps = spec.eps

    def forward(self, x, ctx):
        """x: the residual stream in the compute dtype. Returns y [N, hidden]; the block norms it into the stream."""
        s, ops = self.spec, self.ops
        t = ops.linear(x, self.w_gate)
        return ops.linear(ops.side_gate(t, self.table, s.index * s.dim, ctx.token_ids), self.w_proj)


register_part(TokenSideSpec, TokenSide)
