"""Linear attention with a matrix state per head and request: S <- diag(decay) S + k v^T, o = S^T q.

``GatedLinearAttention``: the decay is a number per key channel that depends on the token,
sigmoid(z)^(1 / tau) with z a low-rank projection of the layer's input plus a bias; q is scaled by
head_dim^-1/2; each head's result is RMS-normed with one gain for all heads and multiplied by silu of
a gate. ``LightningAttention``: a fixed decay per head over silu-activated q, k and v; the heads are
normed together and multiplied by the sigmoid of a gate. In both one product reads the layer's input
(rows [gate | q | k | v], and the decay's inner projection behind them), one kernel walks each
sequence's tokens of the step from the row's float32 state and leaves the state for the next step, and
the norm and gate are the kernel that serves the other recurrent mixers.
"""

from __future__ import annotations

import torch

from ..config.specs import GatedLinearAttentionSpec, LightningAttentionSpec
from .registry import RowState, TensorDecl, register_part


class GatedLinearAttention:
    takes_out_dtype = True      # forward(..., out_dtype=): the dtype of its last product

    @staticmethod
    def tensors(spec: GatedLinearAttentionSpec):
        H, D, Dv, d = spec.n_heads, spec.head_dim, spec.v_dim, spec.hidden
        r = spec.decay_rank or -1
        return {"q": TensorDecl((H * D, d)), "k": TensorDecl((H * D, d)), "v": TensorDecl((H * Dv, d)),
                "g": TensorDecl((H * Dv, d)), "o": TensorDecl((d, H * Dv)), "norm": TensorDecl((Dv,), "vector"),
                "a1": TensorDecl((r, d)), "a2": TensorDecl((H * D, r)), "a2.b": TensorDecl((H * D,), "vector")}

    @staticmethod
    def cache_need(spec: GatedLinearAttentionSpec):
        return RowState((spec.n_heads * spec.head_dim * spec.v_dim,))

    def __init__(self, spec: GatedLinearAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, D, Dv = spec.n_heads, spec.head_dim, spec.v_dim
        self.rank = tensors["a1"].shape[0]
        if tensors["a2"].shape[1] != self.rank:
            raise ValueError(f"the decay's two matrices do not meet: {tuple(tensors['a1'].shape)} and {tuple(tensors['a2'].shape)}")
        self.w_first = torch.cat([tensors["g"], tensors["q"], tensors["k"], tensors["v"], tensors["a1"]], dim=0).contiguous()
        self.cols = (H * Dv, H * Dv + H * D, H * Dv + 2 * H * D)
        self.col_inner = 2 * H * Dv + 2 * H * D
        self.w_a2 = tensors["a2"]
        self.a2_bias = tensors["a2.b"].to(torch.float32).contiguous()
        self.w_o = tensors["o"]
        self.gain = tensors["norm"].to(torch.float32).repeat(H).contiguous()

    def forward(self, x, ctx, slot, write=True, out_dtype=None):
        s, ops = self.spec, self.ops
        first = ops.linear(x, self.w_first)
        inner = first[:, self.col_inner:self.col_inner + self.rank].contiguous()
        z = ops.linear(inner, self.w_a2, out_dtype=torch.float32)
        raw = ops.linear_attention(first, self.cols, s.n_heads, s.head_dim, s.v_dim, float(s.head_dim) ** -0.5, False,
                                   None, z, self.a2_bias, s.tau, slot.state, 0, ctx)
        o = ops.gated_group_norm(raw, first, self.gain, s.n_heads, s.eps, gate_first=False)
        return ops.linear(o, self.w_o, out_dtype=out_dtype)


class LightningAttention:
    takes_out_dtype = True

    @staticmethod
    def tensors(spec: LightningAttentionSpec):
        H, D, Dv, d = spec.n_heads, spec.head_dim, spec.v_dim, spec.hidden
        return {"q": TensorDecl((H * D, d)), "k": TensorDecl((H * D, d)), "v": TensorDecl((H * Dv, d)),
                "g": TensorDecl((H * Dv, d)), "o": TensorDecl((d, H * Dv)), "norm": TensorDecl((H * Dv,), "vector")}

    @staticmethod
    def cache_need(spec: LightningAttentionSpec):
        return RowState((spec.n_heads * spec.head_dim * spec.v_dim,))

    def __init__(self, spec: LightningAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, D, Dv = spec.n_heads, spec.head_dim, spec.v_dim
        self.w_first = torch.cat([tensors["g"], tensors["q"], tensors["k"], tensors["v"]], dim=0).contiguous()
        self.cols = (H * Dv, H * Dv + H * D, H * Dv + 2 * H * D)
        self.w_o = tensors["o"]
        self.gain = tensors["norm"].to(torch.float32).contiguous()
        self.decays = torch.tensor(spec.decays, dtype=torch.float64).to(torch.float32).to(ops.device)

    def forward(self, x, ctx, slot, write=True, out_dtype=None):
        s, ops = self.spec, self.ops
        first = ops.linear(x, self.w_first)
        raw = ops.linear_attention(first, self.cols, s.n_heads, s.head_dim, s.v_dim, 1.0, True, self.decays, None, None,
                                   1.0, slot.state, 0, ctx)
        o = ops.gated_group_norm(raw, first, self.gain, 1, s.eps, gate_first=False, sigmoid=True)
        return ops.linear(o, self.w_o, out_dtype=out_dtype)


register_part(GatedLinearAttentionSpec, GatedLinearAttention)
register_part(LightningAttentionSpec, LightningAttention)
