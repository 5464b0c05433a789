"""Arrangements of a mixer, a feed-forward and their norms into one layer.

"prenorm" (model/qwen/qwen_kv_paged.py:186-189): h = x + mixer(norm1(x));
y = h + ffn(norm2(h)). The residual stream is a float32 tensor updated in place;
each sum is fused into the norm that follows it, so a block returns its last
branch output un-added ("pending") and the next norm adds it.
"""

from __future__ import annotations

from ..config.specs import BlockSpec, DepthAverageSpec
from .registry import TensorDecl, build_part, register_part, tensors_of

_ARRANGEMENTS = {}


def register_arrangement(name: str, cls) -> None:
    _ARRANGEMENTS[name] = cls


def block_tensors(spec: BlockSpec):
    """{full tensor name: TensorDecl} of one layer."""
    out = {}
    for role in spec.ROLES:
        sub = getattr(spec, role)
        if sub is None:
            continue
        for local, decl in tensors_of(sub).items():
            out[_joined(spec.name_of(role), local)] = decl
    return out


def _joined(base: str, local: str) -> str:
    """A part's tensor on disk: the part's name, a dot, the local name; a local name of ""
    is the tensor that carries the part's own name, and one that starts with "/" is a name of the
    whole model (a tensor that several layers share)."""
    if local.startswith("/"):
        return local[1:]
    return f"{base}.{local}" if local else base


def build_block(spec: BlockSpec, weights, ops):
    try:
        cls = _ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown block arrangement {spec.arrangement!r}; "
                       f"known: {sorted(_ARRANGEMENTS)}") from None
    return cls(spec, weights, ops)


def _sub_tensors(spec: BlockSpec, role: str, weights):
    sub = getattr(spec, role)
    return {local: weights[_joined(spec.name_of(role), local)] for local in tensors_of(sub)}


class Normed:
    """What a branch returns when its last projection has already added its output to the
    residual stream and computed the following norm: ``rows`` is that norm's output (a
    tensor, or whatever the kernel set hands the next product in its place)."""
    __slots__ = ("rows",)

    def __init__(self, rows):
        self.rows = rows


class Biased:
    """What a branch returns when its last product's bias is left to whoever adds the result: ``rows`` (float32 or
    the compute dtype) and ``bias`` (float32 [d])."""
    __slots__ = ("rows", "bias")

    def __init__(self, rows, bias):
        self.rows, self.bias = rows, bias


class PreNormBlock:
    chains = True       # forward takes ``nxt``, the block that runs after this one

    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec, self.ops = spec, ops
        self.norm1 = build_part(spec.norm1, _sub_tensors(spec, "norm1", weights), ops)
        self.mixer = build_part(spec.mixer, _sub_tensors(spec, "mixer", weights), ops)
        self.norm2 = build_part(spec.norm2, _sub_tensors(spec, "norm2", weights), ops)
        self.ffn = build_part(spec.ffn, _sub_tensors(spec, "ffn", weights), ops)
        # a step through this layer can be captured into a HIP graph unless one of its parts
        # says otherwise (it reads the host's view of the batch, or syncs with the device)
        self.capturable = all(getattr(p, "capturable", True)
                              for p in (self.norm1, self.mixer, self.norm2, self.ffn))

    def reserve(self, n_positions):
        """Pass the cache's longest row on to the parts that keep something by position."""
        for part in (self.norm1, self.mixer, self.norm2, self.ffn):
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def _branch(self, part, args, residual, norm, consumer):
        """Run a mixer or feed-forward. If the part ends with a projection that it lets the
        block supply (``takes_projection``), the norm after it can be left to the kernel set
        (``fusable``) and the part after that norm takes what the kernel set then returns in
        place of normed rows (``takes_norm_owed``), the part's last product adds to the
        residual stream and prepares the norm itself: one kernel instead of two."""
        ops = self.ops
        if (getattr(part, "takes_projection", False) and norm is not None and hasattr(norm, "fusable")
                and getattr(consumer, "takes_norm_owed", False) and hasattr(ops, "linear_add_norm")):
            gain, eps = norm.fusable()
            return part.forward(*args, project=lambda y, w: Normed(ops.linear_add_norm(y, w, residual, gain, eps)))
        return part.forward(*args)

    @staticmethod
    def _norm(norm, consumer, residual, delta):
        """The sum and the norm before a part. A part that feeds its input to one product of the
        kernel set and nowhere else (``takes_norm_owed``) leaves the layout of that input to the
        kernel set, if the norm can write it so (``free_layout``)."""
        if getattr(norm, "free_layout", False) and getattr(consumer, "takes_norm_owed", False):
            return norm.add_norm(residual, delta, by_tile=True)
        return norm.add_norm(residual, delta)

    def forward(self, residual, pending, ctx, slot, write=True, nxt=None):
        """residual: fp32 [N, hidden], updated in place. pending: the previous block's
        un-added output, None, or a ``Normed`` (already added, and normed by this block's
        first norm). ``nxt``: the block that runs next, if it is of this arrangement.
        Returns this block's feed-forward output, un-added or as a ``Normed``."""
        h = pending.rows if isinstance(pending, Normed) else self._norm(self.norm1, self.mixer, residual, pending)
        a = self._branch(self.mixer, (h, ctx, slot, write), residual, self.norm2, self.ffn)
        h = a.rows if isinstance(a, Normed) else self._norm(self.norm2, self.ffn, residual, a)
        return self._branch(self.ffn, (h, ctx), residual, getattr(nxt, "norm1", None), getattr(nxt, "mixer", None))


class SandwichBlock:
    """x <- x + m * post_norm(gate(h) * branch(h)) with h = norm(x), for the mixer and then for
    the feed-forward (a layer may have none). The gate is sigmoid(W h + b) on the branch's own
    input; the residual stream stays float32. What closes a branch is one kernel: gate, the
    norm of the branch's result, the scaled sum into the stream, and the norm that opens the
    next branch (this block's second, or the next block's first)."""
    chains = True
    # ``Engine.tune`` leaves models with such blocks alone: the one run of the library's tuning pass over
    # such a model (4B-sized layers, a prompt of 2,048 tokens) aborted on the GPU and the cause is not
    # known; every product keeps the library's default solution.
    library_tuning = False

    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec, self.ops = spec, ops
        for role in spec.ROLES:
            sub = getattr(spec, role)
            setattr(self, role, None if sub is None else build_part(sub, _sub_tensors(spec, role, weights), ops))
        if self.ffn is not None and (self.norm2 is None or self.post_norm2 is None):
            raise ValueError("a feed-forward needs the norms before and after it")
        # A branch whose first product reads its input as it comes takes the gate's matrix as further rows of
        # that product (``adopt``): one launch less, and the gate's logits come back beside the branch's result.
        for part, gate in ((self.mixer, self.gate1), (self.ffn, self.gate2)):
            if gate is not None and hasattr(part, "adopt"):
                gate.weight = part.adopt(gate.weight)
        parts = [getattr(self, role) for role in spec.ROLES]
        self.capturable = all(getattr(p, "capturable", True) for p in parts if p is not None)

    def reserve(self, n_positions):
        for role in self.spec.ROLES:
            part = getattr(self, role)
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def _close(self, residual, y, h, gate, post_norm, next_norm):
        """Close a branch whose input was ``h`` and whose result is ``y`` (or (result, gate logits) from a
        branch that has adopted the gate's matrix); returns the rows the next branch reads (None if nothing
        follows in this stream)."""
        ops = self.ops
        logits = bias = None
        if isinstance(y, tuple):
            (y, logits), bias = y, gate.bias
        elif gate is not None:
            logits, bias = ops.linear(h, gate.weight), gate.bias
        more = {}
        if isinstance(y, Biased):                       # the result's own bias, added before the norm
            y, more["y_bias"] = y.rows, y.bias
        if y.dim() == 3 and y.shape[0] == 1:            # float32 sums of a feed-forward that sums in float32
            y = y[0]
        gain, eps = post_norm.fusable()
        follows = next_norm.fusable() if hasattr(next_norm, "fusable") else None
        out = ops.gated_norm_add(residual, y, logits, bias, gain, eps, self.spec.residual_mult,
                                 *(follows or (None, 0.0)), **more)
        if next_norm is not None and follows is None:
            out = next_norm.add_norm(residual, None)
        return out

    def forward(self, residual, pending, ctx, slot, write=True, nxt=None):
        h = pending.rows if isinstance(pending, Normed) else self.norm1.add_norm(residual, pending)
        a = self.mixer.forward(h, ctx, slot, write)
        first_of_next = getattr(nxt, "norm1", None)
        h = self._close(residual, a, h, self.gate1, self.post_norm1, self.norm2 if self.ffn is not None else first_of_next)
        if self.ffn is not None:
            f = self.ffn.forward(h, ctx)
            h = self._close(residual, f, h, self.gate2, self.post_norm2, first_of_next)
        return None if h is None else Normed(h)


class SideInputBlock:
    """Prenorm with a per-layer side input at the end: x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)) (a
    layer may have no feed-forward); then, if the layer has one, x <- x + norm(side(x)) with side reading the
    stream itself. The sum before the side input, and the stream in the compute dtype, are one kernel; the
    norm of the side's result, its sum into the stream and the next block's first norm another."""
    chains = True

    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec, self.ops = spec, ops
        for role in ("norm1", "mixer", "norm2", "ffn", "side"):
            sub = getattr(spec, role)
            setattr(self, role, None if sub is None else build_part(sub, _sub_tensors(spec, role, weights), ops))
        if self.ffn is not None and self.norm2 is None:
            raise ValueError("a feed-forward needs the norm before it")
        parts = (self.norm1, self.mixer, self.norm2, self.ffn, self.side)
        self.capturable = all(getattr(p, "capturable", True) for p in parts if p is not None)

    def reserve(self, n_positions):
        for part in (self.norm1, self.mixer, self.norm2, self.ffn, self.side):
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def forward(self, residual, pending, ctx, slot, write=True, nxt=None):
        ops = self.ops
        h = pending.rows if isinstance(pending, Normed) else self.norm1.add_norm(residual, pending)
        out = self.mixer.forward(h, ctx, slot, write)
        if self.ffn is not None:
            out = self.ffn.forward(self.norm2.add_norm(residual, out), ctx)
        if self.side is None:
            return out
        y = self.side.forward(ops.add_cast(residual, out), ctx)
        first_of_next = getattr(nxt, "norm1", None)
        follows = first_of_next.fusable() if hasattr(first_of_next, "fusable") else None
        rows = ops.gated_norm_add(residual, y, None, None, self.side.gain, self.side.eps, 1.0, *(follows or (None, 0.0)))
        return None if rows is None else Normed(rows)


class DepthAverage:
    """Holds the weights w [index + 2] of what goes on from a layer: sum_j w[j] X_j over the embedding output
    X_0 and the results X_1 .. X_(index+1) of the layers so far."""

    @staticmethod
    def tensors(spec):
        return {"": TensorDecl((spec.index + 2,), "vector")}

    def __init__(self, spec, tensors, ops):
        self.spec, self.weights = spec, tensors[""]


class DepthAverageBlock:
    """Norms on the results only, and a weighted sum over depth at the end: x <- x + norm1(mixer(x));
    x <- x + norm2(ffn(x)) (a layer may have no feed-forward), mixer and feed-forward reading the stream
    itself; that x is the layer's result X_(i+1), and what goes on is sum_j w[j] X_j over the embedding
    output and all layers' results so far. The results are kept in float32 for the length of the step
    (``ctx.carry``: one tensor [layers + 1, N, d] that the first block of a step makes). One kernel norms
    a branch's result, adds it to the stream and casts the sum for the part that reads it next; behind the
    layer's last branch the same kernel files the layer's result, takes the weighted sum and casts it for
    the next layer's mixer."""
    chains = True
    _CARRY = "results by depth"

    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec, self.ops = spec, ops
        built = {}
        for role in ("norm1", "mixer", "norm2", "ffn", "depth"):
            sub = getattr(spec, role)
            built[role] = None if sub is None else build_part(sub, _sub_tensors(spec, role, weights), ops)
        # (the norms are not called norm1 / norm2 here: a block of another arrangement in front of this one
        # would take a ``norm1`` for a norm on this block's input)
        self.post1, self.mixer, self.post2, self.ffn, self.depth = (built[r] for r in ("norm1", "mixer", "norm2", "ffn", "depth"))
        if self.ffn is not None and self.post2 is None:
            raise ValueError("a feed-forward needs the norm behind it")
        if self.depth is None:
            raise ValueError("this arrangement ends with a weighted sum over depth")
        parts = (self.post1, self.mixer, self.post2, self.ffn)
        self.capturable = all(getattr(p, "capturable", True) for p in parts if p is not None)

    def reserve(self, n_positions):
        for part in (self.mixer, self.ffn):
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def forward(self, residual, pending, ctx, slot, write=True, nxt=None):
        ops = self.ops
        depth = self.depth.spec
        # the stream in the compute dtype, for the mixer: the block before has left it, or it is cast here
        # (with whatever that block left un-added)
        if isinstance(pending, Normed):
            x = pending.rows
        elif pending is not None or depth.index != 0:
            x = ops.add_cast(residual, pending)
        if depth.index == 0:
            # the first layer of a step files the embedding output as X_0
            if pending is None:
                ctx.carry[self._CARRY], x = ops.depth_begin(residual, depth.n_layers + 1, cast=True)
            else:
                ctx.carry[self._CARRY] = ops.depth_begin(residual, depth.n_layers + 1)
        kept = ctx.carry[self._CARRY]
        gain, eps = self.post1.fusable()
        # the layer's last branch: its norm, the sum, the filing of the layer's result and the weighted sum over depth
        # are one kernel, which also casts what goes on if the next block reads it as this one does
        last = dict(cast=isinstance(nxt, DepthAverageBlock), depth=(kept, depth.index + 1, self.depth.weights))
        y = self.mixer.forward(x, ctx, slot, write)
        if self.ffn is None:
            rows = ops.norm_add_cast(residual, y, gain, eps, **last)
        else:
            x = ops.norm_add_cast(residual, y, gain, eps, cast=True)
            gain, eps = self.post2.fusable()
            rows = ops.norm_add_cast(residual, self.ffn.forward(x, ctx), gain, eps, **last)
        return None if rows is None else Normed(rows)


register_arrangement("postnorm_depth", DepthAverageBlock)
register_arrangement("prenorm", PreNormBlock)
register_arrangement("prenorm_side", SideInputBlock)
register_arrangement("sandwich", SandwichBlock)

register_part(DepthAverageSpec, DepthAverage)
