"""Grouped-query softmax attention over a sliding window, with what designs put around it: biases of
the projections, an RMS norm of q and k per head or over the whole projection, a rotation over
interleaved pairs with stretched frequencies, values turned by their position and the result turned
back, one mean key and value per block of tokens that lies before the window, a learned sink per head,
kept first keys, a soft cap on the scores, a norm of q and k behind the rotation, values that are the
keys as projected, and a sigmoid gate per head.

One product reads the layer's input: rows [q | k | v]. One kernel adds the biases, norms and turns q
and k, turns the values and writes keys and values to the token's place in the pages; both pools have
heads of ``cache_width`` elements (the larger of the two sizes, padded with zeros, which change neither
scores nor sums). With pooled blocks a second kernel takes the means of the blocks that the step
completes, from the pages, into the slot's pages of means. The paged-attention kernels that serve the
other attention layers then walk the visible means and the window in one softmax.
"""

from __future__ import annotations

import torch

from ..config.specs import WindowAttentionSpec
from .registry import PagedKV, TensorDecl, register_part


def pair_frequencies(position, device):
    """(float32 [dims / 2] evaluated in double precision, dims) of a rotation over pairs; (None, 0) without one."""
    if position is None:
        return None, 0
    return torch.tensor(position.frequencies(), dtype=torch.float64).to(torch.float32).to(device), position.dims


class WindowAttention:
    takes_out_dtype = True      # forward(..., out_dtype=): the dtype of its last product
    offers_raw = True           # forward(..., raw=True): (last product, its bias) with the bias left to the caller

    @staticmethod
    def tensors(spec: WindowAttentionSpec):
        H, G, D, Dv, d = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim, spec.hidden
        t = {"q": TensorDecl((H * D, d)), "k": TensorDecl((G * D, d)), "o": TensorDecl((d, H * Dv))}
        if not spec.tied_values:
            t["v"] = TensorDecl((G * Dv, d))
        if spec.head_gate:
            t["g"] = TensorDecl((H, d))
        if spec.qkv_bias:
            t["q.b"] = TensorDecl((H * D,), "vector")
            t["k.b"] = TensorDecl((G * D,), "vector")
            if not spec.tied_values:
                t["v.b"] = TensorDecl((G * Dv,), "vector")
        if spec.o_bias:
            t["o.b"] = TensorDecl((d,), "vector")
        if spec.qk_norm == "head":
            t["q.norm"] = TensorDecl((D,), "vector")
            t["k.norm"] = TensorDecl((D,), "vector")
        elif spec.qk_norm == "whole":
            t["q.norm"] = TensorDecl((H * D,), "vector")
            t["k.norm"] = TensorDecl((G * D,), "vector")
        if spec.sinks:
            t["sink"] = TensorDecl((H,), "vector")
        return t

    @staticmethod
    def cache_need(spec: WindowAttentionSpec):
        return PagedKV(spec.n_kv_heads, spec.cache_width, spec.window, spec.keep_first if spec.window is not None else 0,
                       spec.pool)

    def __init__(self, spec: WindowAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, G, D, Dv = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim
        # rows [q | k | v | gate]; values that are the keys as projected are the k columns read once more
        rows = [tensors["q"], tensors["k"]] + ([] if spec.tied_values else [tensors["v"]]) + ([tensors["g"]] if spec.head_gate else [])
        self.w_first = torch.cat(rows, dim=0).contiguous()
        self.cols = (0, H * D, H * D if spec.tied_values else H * D + G * D)
        self.col_gate = H * D + G * D + (0 if spec.tied_values else G * Dv)
        self.bias = None
        if spec.qkv_bias:
            parts = [tensors["q.b"], tensors["k.b"]] + ([] if spec.tied_values else [tensors["v.b"]])
            if spec.head_gate:
                parts.append(torch.zeros(H, dtype=parts[0].dtype, device=parts[0].device))
            self.bias = torch.cat(parts).to(torch.float32).contiguous()
        self.w_o = tensors["o"]
        self.o_bias = tensors["o.b"].to(torch.float32).contiguous() if spec.o_bias else None
        self.q_gain, self.k_gain = tensors.get("q.norm"), tensors.get("k.norm")
        self.inv_freq, self.rotary_dim = pair_frequencies(spec.position, ops.device)
        self.value_freq = None
        if spec.value_base is not None:
            m = torch.arange(Dv // 2, dtype=torch.float64)
            self.value_freq = (spec.value_base ** (-2.0 * m / Dv)).to(torch.float32).to(ops.device)
        self.sinks = tensors["sink"].to(torch.float32).contiguous() if spec.sinks else None
        self.magnitude = spec.position.magnitude if spec.position is not None else 1.0
        if spec.head_gate and spec.value_base is not None:
            raise ValueError("a gate per head and values turned back are not combined here")

    def forward(self, x, ctx, slot, write=True, out_dtype=None, raw=False):
        """``raw``: return (product, the output projection's bias or None) and leave the bias to the caller."""
        s, ops = self.spec, self.ops
        H, G, D, Dv, P = s.n_heads, s.n_kv_heads, s.head_dim, s.v_dim, s.cache_width
        if not write:
            raise ValueError("this attention writes the cache slot it reads")
        first = ops.linear(x, self.w_first)
        more = {} if self.magnitude == 1.0 else {"magnitude": self.magnitude}
        q = ops.window_prepare(first, self.cols, H, G, D, Dv, P, self.bias, self.q_gain, self.k_gain, s.qk_norm, s.eps,
                               self.inv_freq, self.rotary_dim, self.value_freq, ctx.positions, ctx.token_rows, slot, **more)
        terms = {}
        if self.sinks is not None:
            terms["sinks"] = self.sinks
        if s.softcap is not None:
            terms["softcap"] = s.softcap
        if s.window is not None and s.keep_first:
            terms["keep_first"] = s.keep_first
        if s.pool:
            ops.pool_blocks(slot, ctx)
            terms["pooled"] = slot
        o = ops.paged_attention(q, slot, ctx, s.scale, s.window, terms=terms or None)
        if s.head_gate:
            o = ops.head_gate(o, H, P, Dv, first[:, self.col_gate:self.col_gate + H])
        elif self.value_freq is not None or P != Dv:
            o = ops.turn_back(o, H, P, Dv, self.value_freq, ctx.positions)
        y = ops.linear(o, self.w_o, out_dtype=out_dtype)
        if raw:
            return y, self.o_bias
        return y if self.o_bias is None else ops.scaled_sum(y, 1.0, None, 0.0, self.o_bias)


register_part(WindowAttentionSpec, WindowAttention)
