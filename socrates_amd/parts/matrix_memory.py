"""A matrix memory per head with exponential gates (mLSTM), carried per request in float32.

With log gates i and f and a running maximum m (0 when a row opens): m' = max(f + m, i),
S <- exp(f + m - m') S + exp(i - m') k v^T, n likewise with k alone, o = S^T q / (max(|n . q|, exp(-m')) + eps').
n rides as one more column of S (a value that is always 1), so the recurrence is linear attention with a
decay per token and head and keys scaled per token: the kernel that serves the other linear-attention
mixers walks it, fed by one kernel that takes the gates, walks the maxima of each sequence's tokens and
prepares q, k and decays in float32. One product reads the layer's input (rows [gate | q | k | v]); the
gates' logits are a product of their own with float32 results. A last kernel divides by the
denominators, norms each head, and applies gain and sigmoid gate.
"""

from __future__ import annotations

import torch

from ..config.specs import MatrixMemorySpec
from .registry import RowState, TensorDecl, register_part


class MatrixMemory:
    @staticmethod
    def tensors(spec: MatrixMemorySpec):
        H, D, Dv, d = spec.n_heads, spec.head_dim, spec.v_dim, spec.hidden
        return {"q": TensorDecl((H * D, d)), "k": TensorDecl((H * D, d)), "v": TensorDecl((H * Dv, d)),
                "g": TensorDecl((H * Dv, d)), "o": TensorDecl((d, H * Dv)), "norm": TensorDecl((H * Dv,), "vector"),
                "i": TensorDecl((H, d)), "i.b": TensorDecl((H,), "vector"),
                "f": TensorDecl((H, d)), "f.b": TensorDecl((H,), "vector")}

    @staticmethod
    def cache_need(spec: MatrixMemorySpec):
        # per head [D, Dv + 1]: S with n as its last column; behind all heads the running maxima
        return RowState((spec.n_heads * spec.head_dim * (spec.v_dim + 1) + spec.n_heads,))

    def __init__(self, spec: MatrixMemorySpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, D, Dv = spec.n_heads, spec.head_dim, spec.v_dim
        self.w_first = torch.cat([tensors["g"], tensors["q"], tensors["k"], tensors["v"]], dim=0).contiguous()
        self.cols = (H * Dv, H * Dv + H * D, H * Dv + 2 * H * D)
        self.w_gates = torch.cat([tensors["i"], tensors["f"]], dim=0).contiguous()
        self.gate_bias = torch.cat([tensors["i.b"], tensors["f.b"]]).to(torch.float32).contiguous()
        self.w_o = tensors["o"]
        self.gain = tensors["norm"].to(torch.float32).contiguous()
        self.offset_max = H * D * (Dv + 1)

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        H, D, Dv = s.n_heads, s.head_dim, s.v_dim
        first = ops.linear(x, self.w_first)
        gates = ops.linear(x, self.w_gates, out_dtype=torch.float32)
        prep, maxima = ops.memory_gates(gates, self.gate_bias, s.gate_cap, first, self.cols, H, D, float(D) ** -0.5,
                                        slot.state, self.offset_max, ctx)
        raw = ops.linear_attention(first, self.cols, H, D, Dv + 1, 1.0, False, None, None, None, 1.0, slot.state, 0, ctx,
                                   prepared=prep, ones=1)
        o = ops.memory_finish(raw, maxima, first, self.gain, H, Dv, s.eps, s.den_eps)
        return ops.linear(o, self.w_o)


register_part(MatrixMemorySpec, MatrixMemory)
