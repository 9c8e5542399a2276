"""Routed experts: a mixture of small clamped gated feed-forwards of which each token uses a few,
chosen among groups of experts, beside one that every token uses.

Router logits and everything behind them up to the weights are float32. The tokens of a step are
sorted by expert on the device, the two products run per expert over its run of tokens, and a
token's weighted sum is taken in float32 and handed to the residual sum as it is; nothing waits for
the host, so steps with such a layer can be captured.
"""

from __future__ import annotations

import torch

from ..config.specs import RoutedExpertsSpec
from .registry import TensorDecl, build_part, register_part, tensors_of


class RoutedExperts:
    @staticmethod
    def tensors(spec: RoutedExpertsSpec):
        t = {"router": TensorDecl((spec.n_experts, spec.hidden))}
        if spec.corrected:
            t["correction"] = TensorDecl((spec.n_experts,), "vector")
        for e in range(spec.n_experts):
            for local, decl in tensors_of(spec.expert).items():
                t[f"e{e}.{local}"] = decl
        if spec.shared is not None:
            for local, decl in tensors_of(spec.shared).items():
                t[f"shared.{local}"] = decl
        return t

    def __init__(self, spec: RoutedExpertsSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        E = spec.n_experts
        self.w_router = tensors["router"]
        self.correction = tensors.get("correction")
        # [E, gate | up, hidden] and [E, hidden, ff]: one operand each for the products per expert
        self.w_gate_up = torch.stack([torch.cat([tensors[f"e{e}.gate"], tensors[f"e{e}.up"]], dim=0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors[f"e{e}.down"] for e in range(E)]).contiguous()
        self.shared = None
        if spec.shared is not None:
            self.shared = build_part(spec.shared, {k[len("shared."):]: v for k, v in tensors.items() if k.startswith("shared.")}, ops)

    def forward(self, x, ctx=None):
        s, ops = self.spec, self.ops
        logits = ops.linear(x, self.w_router, out_dtype=torch.float32)
        experts, weights = ops.moe_route(logits, self.correction, s.top, s.n_groups, s.keep_groups, s.renorm_eps)
        extra = self.shared.forward(x) if self.shared is not None else None
        y = ops.moe_experts(x, experts, weights, self.w_gate_up, self.w_down, s.expert.limit, s.expert.slope, extra)
        return y.unsqueeze(0)        # float32 sums: the residual sum takes them as they are


register_part(RoutedExpertsSpec, RoutedExperts)
