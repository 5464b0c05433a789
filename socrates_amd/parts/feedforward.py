"""SwiGLU feed-forward: y = Wd((Wu x) * silu(Wg x)), no bias
(model/qwen/qwen_kv_cont.py:250-266). silu(z) = z * sigmoid(z), on the gate."""

from __future__ import annotations

import torch

from ..config.specs import ClampedGLUSpec, GeluGLUSpec, ReluSquaredSpec, SigmoidGateSpec, SwiGLUSpec
from .registry import TensorDecl, register_part


class SwiGLU:
    @staticmethod
    def tensors(spec: SwiGLUSpec):
        gate, up, down = spec.names
        return {gate: TensorDecl((spec.intermediate, spec.hidden)),
                up: TensorDecl((spec.intermediate, spec.hidden)),
                down: TensorDecl((spec.hidden, spec.intermediate))}

    def __init__(self, spec: SwiGLUSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        # One operand for gate and up. Where the width allows, their rows alternate in blocks
        # of 16 (16 gate rows, the 16 up rows of the same columns, ...): a workgroup of the
        # decode product then holds both and applies the activation itself.
        gate, up = tensors[spec.names[0]], tensors[spec.names[1]]
        ff = spec.intermediate
        self.interleave = 16 if ff % 16 == 0 else 0
        if self.interleave:
            self.w_gate_up = torch.stack([gate.view(ff // 16, 16, -1), up.view(ff // 16, 16, -1)],
                                         dim=1).reshape(2 * ff, -1).contiguous()
        else:
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors[spec.names[2]]
        # (the activation goes to a product and nowhere else: the kernel set may lay it out as it likes)
        self._free_layout = {"by_tile": True} if getattr(ops, "rows_by_tile", None) is not None else {}

    takes_projection = True     # the block may supply the last product
    takes_norm_owed = True      # x goes to one product only

    def rows_as_they_are(self):
        """The activation goes to a product that reads plain rows (a caller's own ``project``): keep the rows' layout."""
        self._free_layout = {}

    def forward(self, x, ctx=None, project=None):
        act = self.ops.linear_swiglu(x, self.w_gate_up, self.interleave, **self._free_layout)
        if project is not None:
            return project(act, self.w_down)
        # the block's next norm adds this output to the residual: partial sums are welcome
        return self.ops.linear(act, self.w_down, allow_partial=True)


class ClampedGLU:
    """y = Wd(g * sigmoid(slope * g) * (u + 1)), g = min(Wg x, limit), u = clamp(Wu x, +-limit)."""

    @staticmethod
    def tensors(spec: ClampedGLUSpec):
        return {"gate": TensorDecl((spec.intermediate, spec.hidden)),
                "up": TensorDecl((spec.intermediate, spec.hidden)),
                "down": TensorDecl((spec.hidden, spec.intermediate))}

    def __init__(self, spec: ClampedGLUSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        # one operand for gate and up: rows [gate | up]
        self.w_gate_up = torch.cat([tensors["gate"], tensors["up"]], dim=0).contiguous()
        self.w_down = tensors["down"]
        self.adopted = 0

    def adopt(self, w):
        """Take ``w`` [n, hidden] as further rows of the first product; ``forward`` then returns (y, x w^T).
        Returns the rows as they now lie (a view), for whoever held ``w``."""
        self.w_gate_up = torch.cat([self.w_gate_up, w], dim=0).contiguous()
        self.adopted = w.shape[0]
        return self.w_gate_up[2 * self.spec.intermediate:]

    def forward(self, x, ctx=None):
        ff = self.spec.intermediate
        both = self.ops.linear(x, self.w_gate_up)
        act = self.ops.glu_clamped(both, self.spec.limit, self.spec.slope, ff)
        y = self.ops.linear(act, self.w_down)
        return (y, both[:, 2 * ff:]) if self.adopted else y


class ReluSquared:
    """y = Wd(relu(Wu x)^2)."""

    @staticmethod
    def tensors(spec: ReluSquaredSpec):
        return {"up": TensorDecl((spec.intermediate, spec.hidden)), "down": TensorDecl((spec.hidden, spec.intermediate))}

    def __init__(self, spec: ReluSquaredSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.w_up, self.w_down = tensors["up"], tensors["down"]

    def forward(self, x, ctx=None):
        return self.ops.linear(self.ops.relu_squared(self.ops.linear(x, self.w_up)), self.w_down)


class GeluGLU:
    """y = Wd(gelu_tanh(Wg x) * (Wu x))."""

    @staticmethod
    def tensors(spec: GeluGLUSpec):
        return {"gate": TensorDecl((spec.intermediate, spec.hidden)), "up": TensorDecl((spec.intermediate, spec.hidden)),
                "down": TensorDecl((spec.hidden, spec.intermediate))}

    def __init__(self, spec: GeluGLUSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.w_gate_up = torch.cat([tensors["gate"], tensors["up"]], dim=0).contiguous()      # rows [gate | up]
        self.w_down = tensors["down"]

    def forward(self, x, ctx=None):
        act = self.ops.glu_gelu(self.ops.linear(x, self.w_gate_up), self.spec.intermediate)
        return self.ops.linear(act, self.w_down)


class SigmoidGate:
    """Holds W [dim, dim] and b [dim] of sigmoid(W h + b); the block computes it where it closes
    a branch."""

    @staticmethod
    def tensors(spec: SigmoidGateSpec):
        return {"": TensorDecl((spec.dim, spec.dim)), "b": TensorDecl((spec.dim,), "vector")}

    def __init__(self, spec: SigmoidGateSpec, tensors, ops):
        self.spec, self.weight, self.bias = spec, tensors[""], tensors["b"]


register_part(SwiGLUSpec, SwiGLU)
register_part(ClampedGLUSpec, ClampedGLU)
register_part(SigmoidGateSpec, SigmoidGate)
register_part(ReluSquaredSpec, ReluSquared)
register_part(GeluGLUSpec, GeluGLU)
