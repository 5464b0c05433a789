"""Differential attention: two softmax maps per head over the same values, the second subtracted with one
weight for the layer, over a window that keeps the first tokens visible.

The two maps are served as attention heads of their own by the paged-attention kernels that serve the
other attention layers: map m of key/value head g is cache head 2 g + m (the keys lie so in the
projection already; the values' rows are doubled once at load, so each map's cache head has the values
beside its keys), and the query projection's rows are reordered once at load to (kv head, map, query
head of the group), so that plain grouped-query indexing pairs every query map with its key map. One
product reads the layer's input (rows [q | k | v]); one kernel adds the biases, turns q and k and
writes the pages; after the attention one kernel takes a1 - lambda a2 per head, divides by its root
mean square and scales. A layer without projections of keys and values reads another such layer's
cache slot with queries, mask and constants of its own.
"""

from __future__ import annotations

import math

import torch

from ..config.specs import DifferentialAttentionSpec
from .block import Biased
from .registry import PagedKV, TensorDecl, register_part
from .window_attention import pair_frequencies


class DifferentialAttention:
    @staticmethod
    def tensors(spec: DifferentialAttentionSpec):
        H, G, D, Dv, d = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim, spec.hidden
        t = {"q": TensorDecl((H * 2 * D, d)), "q.b": TensorDecl((H * 2 * D,), "vector"),
             "o": TensorDecl((d, H * Dv)), "o.b": TensorDecl((d,), "vector")}
        if spec.own_kv:
            t.update({"k": TensorDecl((G * 2 * D, d)), "k.b": TensorDecl((G * 2 * D,), "vector"),
                      "v": TensorDecl((G * Dv, d)), "v.b": TensorDecl((G * Dv,), "vector")})
        for name in ("lq1", "lk1", "lq2", "lk2"):
            t[name] = TensorDecl((D,), "vector")
        return t

    @staticmethod
    def cache_need(spec: DifferentialAttentionSpec):
        window, keep = spec.cache_mask
        return PagedKV(2 * spec.n_kv_heads, spec.cache_width, window, keep)

    def __init__(self, spec: DifferentialAttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        H, G, D, Dv, d = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_dim, spec.hidden
        R = H // G
        # query rows from (kv head, query head of the group, map) to (kv head, map, query head of the group)
        w_q = tensors["q"].view(G, R, 2, D, d).permute(0, 2, 1, 3, 4).reshape(2 * H * D, d)
        b_q = tensors["q.b"].view(G, R, 2, D).permute(0, 2, 1, 3).reshape(2 * H * D)
        self.w_q = w_q.contiguous()
        self.bias_q = b_q.to(torch.float32).contiguous()
        if spec.own_kv:
            w_v = tensors["v"].view(G, 1, Dv, d).expand(G, 2, Dv, d).reshape(2 * G * Dv, d)
            b_v = tensors["v.b"].view(G, 1, Dv).expand(G, 2, Dv).reshape(2 * G * Dv)
            self.w_first = torch.cat([w_q, tensors["k"], w_v], dim=0).contiguous()
            self.w_q = self.w_first[:2 * H * D]
            self.bias = torch.cat([b_q, tensors["k.b"], b_v]).to(torch.float32).contiguous()
        self.cols = (0, 2 * H * D, 2 * H * D + 2 * G * D)
        self.w_o = tensors["o"]
        self.o_bias = tensors["o.b"].to(torch.float32).contiguous()
        f64 = {n: tensors[n].to(torch.float64) for n in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = (math.exp(float((f64["lq1"] * f64["lk1"]).sum())) - math.exp(float((f64["lq2"] * f64["lk2"]).sum()))
                    + spec.diff)
        self.inv_freq, self.rotary_dim = pair_frequencies(spec.position, ops.device)
        self.magnitude = spec.position.magnitude if spec.position is not None else 1.0
        self.terms = {"keep_first": spec.keep_first} if spec.window is not None and spec.keep_first else None

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        H, G, D, Dv, P = s.n_heads, s.n_kv_heads, s.head_dim, s.v_dim, s.cache_width
        if write != s.own_kv:
            raise ValueError("a layer with projections of keys and values writes its cache slot, one without reads another's")
        more = {} if self.magnitude == 1.0 else {"magnitude": self.magnitude}
        if write:
            first = ops.linear(x, self.w_first)
            q = ops.window_prepare(first, self.cols, 2 * H, 2 * G, D, Dv, P, self.bias, None, None, None, s.eps, self.inv_freq,
                                   self.rotary_dim, None, ctx.positions, ctx.token_rows, slot, **more)
        else:
            first = ops.linear(x, self.w_q)
            q = ops.window_prepare(first, (0, 0, 0), 2 * H, 0, D, Dv, P, self.bias_q, None, None, None, s.eps, self.inv_freq,
                                   self.rotary_dim, None, ctx.positions, ctx.token_rows, None, **more)
        o = ops.paged_attention(q, slot, ctx, s.scale, s.window, terms=self.terms)
        o = ops.diff_combine(o, H, G, P, Dv, self.lam, s.eps, 1.0 - s.diff)
        # the last product in float32 with its bias apart: the block adds it where it norms the result
        return Biased(ops.linear(o, self.w_o, out_dtype=torch.float32), self.o_bias)


register_part(DifferentialAttentionSpec, DifferentialAttention)
