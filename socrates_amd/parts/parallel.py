"""Two mixers side by side on the same input, their results scaled and added in float32. Each keeps
its own cache or state: the mixer's need is the pair of theirs, its slot the pair of their slots."""

from __future__ import annotations

import torch

from ..config.specs import ParallelMixerSpec
from .registry import build_part, impl_of, register_part, tensors_of


class ParallelMixer:
    @staticmethod
    def tensors(spec: ParallelMixerSpec):
        out = {}
        for side in ("left", "right"):
            for local, decl in tensors_of(getattr(spec, side)).items():
                if local.startswith("/"):
                    out[local] = decl
                else:
                    out[f"{side}.{local}" if local else side] = decl
        return out

    @staticmethod
    def cache_need(spec: ParallelMixerSpec):
        return tuple(impl_of(m).cache_need(m) for m in (spec.left, spec.right))

    def __init__(self, spec: ParallelMixerSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        sides = []
        for side in ("left", "right"):
            sub = getattr(spec, side)
            mine = {}
            for local in tensors_of(sub):
                key = local if local.startswith("/") else (f"{side}.{local}" if local else side)
                mine[local] = tensors[key]
            sides.append(build_part(sub, mine, ops))
        self.left, self.right = sides
        self.capturable = all(getattr(p, "capturable", True) for p in sides)

    def reserve(self, n_positions):
        for part in (self.left, self.right):
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def forward(self, x, ctx, slot, write=True):
        s, ops = self.spec, self.ops
        # a side that says so hands over its last product in float32 (and its bias apart): the scaled sum is
        # then taken of unrounded results
        bias = None
        wide = {"out_dtype": torch.float32}
        if getattr(self.left, "offers_raw", False):
            a, bias = self.left.forward(x, ctx, slot[0], write, raw=True, **wide)
        else:
            a = self.left.forward(x, ctx, slot[0], write, **(wide if getattr(self.left, "takes_out_dtype", False) else {}))
        b = self.right.forward(x, ctx, slot[1], write, **(wide if getattr(self.right, "takes_out_dtype", False) else {}))
        return ops.scaled_sum(a, s.left_scale, b, s.right_scale, bias)


register_part(ParallelMixerSpec, ParallelMixer)
