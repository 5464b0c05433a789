"""Routed experts: a mixture of small gated feed-forwards (clamped, or with a plain silu gate) of which each
token uses a few, chosen among groups of experts, beside one that every token uses (unweighted, or times a
sigmoid gate per token).

Router logits and everything behind them up to the weights are float32. The tokens of a step are
sorted by expert on the device, the two products run per expert over its run of tokens, and a
token's weighted sum is taken in float32 and handed to the residual sum as it is; nothing waits for
the host, so steps with such a layer can be captured.
"""

from __future__ import annotations

import torch

from ..config.specs import ClampedGLUSpec, RoutedExpertsSpec, SwiGLUSpec
from .registry import TensorDecl, build_part, register_part, tensors_of

NO_LIMIT = 3.0e38        # a clamp that never bites: what the products per expert get for a plain silu gate


def _expert_form(expert):
    """((gate, up, down): an expert's local tensor names, (limit, slope, shift) of g sigmoid(slope g) (u + shift))."""
    if isinstance(expert, SwiGLUSpec):
        return expert.names, (NO_LIMIT, 1.0, 0.0)
    if isinstance(expert, ClampedGLUSpec):
        return ("gate", "up", "down"), (expert.limit, expert.slope, 1.0)
    raise TypeError(f"routed experts of {type(expert).__name__}: a clamped or a silu-gated feed-forward")


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
        if spec.shared_gate:
            t["shared.sg"] = TensorDecl((1, spec.hidden))
        return t

    def __init__(self, spec: RoutedExpertsSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        E = spec.n_experts
        # (the shared expert's gate is one more row of the router's product)
        self.w_router = torch.cat([tensors["router"], tensors["shared.sg"]], dim=0).contiguous() if spec.shared_gate else tensors["router"]
        self.correction = tensors.get("correction")
        (gate, up, down), self.form = _expert_form(spec.expert)
        # [E, gate | up, hidden] and [E, hidden, ff]: one operand each for the products per expert
        self.w_gate_up = torch.stack([torch.cat([tensors[f"e{e}.{gate}"], tensors[f"e{e}.{up}"]], dim=0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors[f"e{e}.{down}"] for e in range(E)]).contiguous()
        self.shared = None
        if spec.shared is not None:
            own = {k[len("shared."):]: v for k, v in tensors.items() if k.startswith("shared.") and k != "shared.sg"}
            self.shared = build_part(spec.shared, own, ops)
            if hasattr(self.shared, "rows_as_they_are"):
                self.shared.rows_as_they_are()

    def forward(self, x, ctx=None):
        s, ops = self.spec, self.ops
        E = s.n_experts
        logits = ops.linear(x, self.w_router, out_dtype=torch.float32)
        plain = s.scoring == "softmax" and s.group_top == 1 and s.scale == 1.0 and not s.shared_gate
        how = {} if plain else dict(scoring=s.scoring, group_top=s.group_top, scale=s.scale)
        experts, weights = ops.moe_route(logits[:, :E] if s.shared_gate else logits, self.correction, s.top, s.n_groups,
                                         s.keep_groups, s.renorm_eps, **how)
        extra = None
        if self.shared is not None and getattr(self.shared, "takes_projection", False):
            # (a feed-forward that would hand partial sums to a norm: here its last product is whole)
            extra = self.shared.forward(x, project=lambda act, w: ops.linear(act, w))
        elif self.shared is not None:
            extra = self.shared.forward(x)
        limit, slope, shift = self.form
        more = {}
        if shift != 1.0:
            more["shift"] = shift
        if s.shared_gate:
            more["extra_gate"] = logits[:, E]
        y = ops.moe_experts(x, experts, weights, self.w_gate_up, self.w_down, limit, slope, extra, **more)
        return y.unsqueeze(0)        # float32 sums: the residual sum takes them as they are


register_part(RoutedExpertsSpec, RoutedExperts)
