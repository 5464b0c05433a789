"""Typed configuration of Berelorn (``"architecture": "Berelorn"``).

A decoder whose layers differ: ``layers`` lists them, each with the ``type`` of its mixer (``mlstm``: a
matrix memory per head with exponential gates; ``attention``: differential attention, two softmax maps
per head over a window that keeps the first tokens, with biases and a stretched rotation over
interleaved pairs, which a layer may run on the keys and values that another such layer caches
(``kv_from``); ``attention_2``: causal attention whose values are the keys as projected, with q and k
normed behind the rotation, soft-capped scores and a sigmoid gate per head), the mixer's sizes, and its
feed-forward (``moe``: silu-gated experts chosen by sigmoid scores among groups, beside a shared expert
with a gate per token; or none). Every sublayer has a norm before it and a norm on its result. Tensor
names: layer i's start with ``l<i>.``, the mixer's with ``l<i>.mix.``, the feed-forward's with
``l<i>.mlp.``; the output head is the embedding table.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Tuple

from .mitisun import _freeze, _positive_int, _thaw
from .qwen3 import ConfigError
from .specs import (BlockSpec, DifferentialAttentionSpec, MatrixMemorySpec, ModelPlan, PairRopeSpec, RMSNormSpec,
                    RoutedExpertsSpec, RunStep, SwiGLUSpec, WindowAttentionSpec)
from .tedulorn import _number

_NAMES = (("norm1", "norm1"), ("post_norm1", "norm1b"), ("mixer", "mix"), ("norm2", "norm2"), ("post_norm2", "norm2b"),
          ("ffn", "mlp"))
_GLU_NAMES = ("gate", "up", "down")
_MIXER_KEYS = {
    "mlstm": ("heads", "dim", "vdim", "gate_cap"),
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "diff"),
    "attention_2": ("heads", "kv_heads", "dim", "scale"),
}


def _check_rotation(where, rot, dim):
    if rot is None:
        return
    if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
        raise ConfigError(f"{where}: rot needs base and dims")
    dims = rot["dims"]
    if not isinstance(dims, int) or isinstance(dims, bool) or dims < 0 or dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims must be even and at most the head size {dim}, found {dims!r}")
    if not _number(where, "rot.base", rot["base"]) > 1:
        raise ConfigError(f"{where}: rot.base must lie above 1")
    sc = rot.get("scaling")
    if sc is not None:
        for k in ("factor", "original", "fast", "slow"):
            if not isinstance(sc, dict) or k not in sc:
                raise ConfigError(f"{where}: rot.scaling needs factor, original, fast and slow")
            _number(where, f"rot.scaling.{k}", sc[k])


def _check_mask(where, mask):
    if mask is None:
        return
    if not isinstance(mask, dict):
        raise ConfigError(f"{where}: mask needs size")
    _positive_int(where, "mask.size", mask.get("size"))
    kf = mask.get("keep_first", 0)
    if not isinstance(kf, int) or isinstance(kf, bool) or kf < 0:
        raise ConfigError(f"{where}: mask.keep_first must be a whole number, not negative, found {kf!r}")


def _position(rot):
    if rot is None or not rot["dims"]:
        return None
    sc = rot.get("scaling")
    ramp = None if sc is None else tuple(float(sc[k]) for k in ("factor", "original", "fast", "slow"))
    return PairRopeSpec(dims=rot["dims"], base=float(rot["base"]), ramp=ramp)


@dataclass(frozen=True)
class BerelornConfig:
    vocab: int
    width: int
    layers: Tuple[tuple, ...]         # as config.json lists them (validated, frozen)
    norm_eps: float
    embedding_scale: float
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Berelorn"

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "BerelornConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing} (required for Berelorn)")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["norm"], dict) or not d["norm"].get("eps", 0) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("layers must list at least one layer")
        scale = 1.0
        if d.get("embedding") is not None:
            scale = _number("config", "embedding.scale", (d["embedding"] or {}).get("scale", 1.0))
        layers = []
        for i, layer in enumerate(d["layers"]):
            where = f"layer {i}"
            kind = layer.get("type")
            if kind not in _MIXER_KEYS:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {sorted(_MIXER_KEYS)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where}: no mixer sizes")
            lacking = [k for k in _MIXER_KEYS[kind] if k not in m]
            if lacking:
                raise ConfigError(f"{where} ({kind}): mixer lacks {lacking}")
            for k in ("heads", "kv_heads", "dim", "vdim"):
                if k in m:
                    _positive_int(where, k, m[k])
            if kind == "mlstm":
                _number(where, "gate_cap", m["gate_cap"])
            else:
                _number(where, "scale", m["scale"])
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: {m['heads']} heads do not divide into {m['kv_heads']} kv heads")
                _check_rotation(where, m.get("rot"), m["dim"])
            if kind == "attention":
                _number(where, "diff", m["diff"], positive=False)
                _check_mask(where, m.get("mask"))
                j = m.get("kv_from")
                if j is not None:
                    if not isinstance(j, int) or isinstance(j, bool) or not 0 <= j < i:
                        raise ConfigError(f"{where}: kv_from names an earlier layer, found {j!r}")
                    other = d["layers"][j]
                    if other.get("type") != "attention" or (other.get("mixer") or {}).get("kv_from") is not None:
                        raise ConfigError(f"{where}: kv_from {j} is not an attention layer with keys and values of its own")
                    om = other["mixer"]
                    if any(om.get(k) != m.get(k) for k in ("heads", "kv_heads", "dim", "vdim", "rot")):
                        raise ConfigError(f"{where}: head counts, sizes and rotation must equal those of layer {j}, "
                                          "whose keys and values it reads")
            if kind == "attention_2":
                if m.get("vdim", m["dim"]) != m["dim"]:
                    raise ConfigError(f"{where}: the values are the keys, so vdim equals dim")
                if m.get("softcap") is not None:
                    _number(where, "softcap", m["softcap"])
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"{where}: feed-forward kind {mlp.get('kind')!r} is not known (moe)")
                _positive_int(where, "mlp.expert.ff", (mlp.get("expert") or {}).get("ff"))
                if mlp.get("shared") is not None:
                    _positive_int(where, "mlp.shared.ff", mlp["shared"].get("ff"))
                r = mlp.get("router")
                if not isinstance(r, dict):
                    raise ConfigError(f"{where}: mlp.router is missing")
                E = _positive_int(where, "router.experts", r.get("experts"))
                top = _positive_int(where, "router.top", r.get("top"))
                if r.get("scale") is not None:
                    _number(where, "router.scale", r["scale"], positive=False)
                g = r.get("groups") or {"count": 1, "keep": 1}
                count = _positive_int(where, "router.groups.count", g.get("count"))
                keep = _positive_int(where, "router.groups.keep", g.get("keep"))
                if top > E or E % count or keep > count or keep * (E // count) < top:
                    raise ConfigError(f"{where}: {top} of {E} experts from {keep} of {count} groups is not possible")
            layers.append(json.loads(json.dumps(layer)))       # a copy of plain values
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(vocab=d["vocab"], width=d["width"], layers=tuple(_freeze(x) for x in layers),
                   norm_eps=float(d["norm"]["eps"]), embedding_scale=scale, eos_token_ids=eos_ids,
                   architecture=d.get("architecture", "Berelorn"))

    @classmethod
    def from_json(cls, path) -> "BerelornConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    # ---- writing -----------------------------------------------------------------
    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
               "layers": [_thaw(x) for x in self.layers], "norm": {"eps": self.norm_eps},
               "vocab": self.vocab, "width": self.width}
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ---- the layer recipe -------------------------------------------------------------
    def _mixer(self, i, layers):
        d, eps = self.width, self.norm_eps
        layer = layers[i]
        m = layer["mixer"]
        if layer["type"] == "mlstm":
            return MatrixMemorySpec(hidden=d, n_heads=m["heads"], head_dim=m["dim"], v_dim=m["vdim"],
                                    gate_cap=float(m["gate_cap"]), eps=eps)
        if layer["type"] == "attention_2":
            return WindowAttentionSpec(hidden=d, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"], v_dim=m["dim"],
                                       scale=float(m["scale"]), eps=eps, qk_norm="turned", position=_position(m.get("rot")),
                                       tied_values=True, softcap=None if m.get("softcap") is None else float(m["softcap"]),
                                       head_gate=True)
        # the cache slot holds what the widest mask among its readers can see
        writer = m["kv_from"] if m.get("kv_from") is not None else i
        masks = [x["mixer"].get("mask") for j, x in enumerate(layers)
                 if x["type"] == "attention" and (j == writer or x["mixer"].get("kv_from") == writer)]
        cache_window = None if any(k is None for k in masks) else max(k["size"] for k in masks)
        cache_keep = 0 if cache_window is None else max(k.get("keep_first", 0) for k in masks)
        mask = m.get("mask")
        return DifferentialAttentionSpec(
            hidden=d, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"], v_dim=m["vdim"], scale=float(m["scale"]),
            eps=eps, diff=float(m["diff"]), position=_position(m.get("rot")), window=None if mask is None else mask["size"],
            keep_first=0 if mask is None else mask.get("keep_first", 0), own_kv=m.get("kv_from") is None,
            cache_window=cache_window, cache_keep_first=cache_keep)

    def _ffn(self, mlp):
        d = self.width
        if mlp is None:
            return None
        r = mlp["router"]
        g = r.get("groups") or {"count": 1, "keep": 1}
        shared = mlp.get("shared")
        return RoutedExpertsSpec(
            hidden=d, n_experts=r["experts"], top=r["top"], expert=SwiGLUSpec(d, mlp["expert"]["ff"], _GLU_NAMES),
            n_groups=g["count"], keep_groups=g["keep"], shared=None if shared is None else SwiGLUSpec(d, shared["ff"], _GLU_NAMES),
            corrected=False, scoring="sigmoid", group_top=2, scale=float(r.get("scale", 1.0) if r.get("scale") is not None else 1.0),
            shared_gate=shared is not None)

    def plan(self) -> ModelPlan:
        d, eps = self.width, self.norm_eps
        layers = [_thaw(x) for x in self.layers]
        norm = RMSNormSpec(d, eps, tensor="")
        blocks, order, ignorable = [], [], []
        for i, layer in enumerate(layers):
            ffn = self._ffn(layer.get("mlp"))
            if ffn is None:                 # (a file may hold the norms of a feed-forward that the layer lacks)
                ignorable += [f"l{i}.norm2", f"l{i}.norm2b"]
            blocks.append(BlockSpec(mixer=self._mixer(i, layers), ffn=ffn, norm1=norm, post_norm1=norm,
                                    norm2=None if ffn is None else norm, post_norm2=None if ffn is None else norm,
                                    prefix=f"l{i}.", names=_NAMES, arrangement="sandwich"))
            j = layer["mixer"].get("kv_from") if layer["type"] == "attention" else None
            order.append(RunStep(layer=i, cache=i, write=True) if j is None else RunStep(layer=i, cache=j, write=False))
        return ModelPlan(
            architecture=self.architecture, vocab_size=self.vocab, hidden=d, layers=tuple(blocks), order=tuple(order),
            final_norm=norm, embedding_name="embed", final_norm_prefix="final.norm", head_name=None,
            eos_token_ids=self.eos_token_ids, ignorable=tuple(ignorable), embedding_scale=self.embedding_scale)

    # ---- byte and flop counts ---------------------------------------------------------
    def _shares(self, plan, of):
        return {f"l{i}.mlp.e": of(block.ffn) for i, block in enumerate(plan.layers) if isinstance(block.ffn, RoutedExpertsSpec)}

    def _weighted_elements(self, share_of, skip=("embed",)):
        from ..parts import expected_tensors
        plan = self.plan()
        share = self._shares(plan, share_of)
        total = 0.0
        for name, decl in expected_tensors(plan).items():
            if name in skip or decl.kind != "matrix":
                continue
            n = 1
            for s in decl.shape:
                n *= max(s, 1)
            total += n * next((f for p, f in share.items() if name.startswith(p)), 1.0)
        return total

    def step_weight_bytes(self, batch: int, item: int) -> int:
        """Bytes of weights that a decode step of ``batch`` tokens reads if its tokens choose their experts
        independently and evenly (of E experts, E (1 - (1 - top / E)^batch) on average); the head is the
        embedding table, read whole."""
        body = self._weighted_elements(lambda f: 1.0 - (1.0 - f.top / f.n_experts) ** batch)
        return int((body + self.vocab * self.width) * item)

    def step_cache_bytes(self, batch: int, context: int, item: int) -> int:
        """Bytes of cache and state that a decode step of ``batch`` requests behind ``context`` tokens reads."""
        total = 0
        for block in self.plan().layers:
            m = block.mixer
            if isinstance(m, MatrixMemorySpec):
                total += 4 * m.n_heads * m.head_dim * (m.v_dim + 1)
            elif isinstance(m, DifferentialAttentionSpec):
                seen = context if m.window is None else min(context, m.window + m.keep_first)
                total += item * 2 * 2 * m.n_kv_heads * m.cache_width * seen
            else:
                total += item * 2 * m.n_kv_heads * m.cache_width * context
        return batch * total

    def prefill_flops(self, tokens: int) -> float:
        """Multiply-adds times two of one prompt of ``tokens`` tokens from position 0: every matrix a token uses
        (of the experts a token's share; the head at one position), attention scores and sums over what each
        token sees, and the recurrence (per token and head, state size times four)."""
        flops = 2.0 * tokens * self._weighted_elements(lambda f: f.top / f.n_experts) + 2.0 * self.vocab * self.width
        for block in self.plan().layers:
            m = block.mixer
            if isinstance(m, MatrixMemorySpec):
                flops += 4.0 * tokens * m.n_heads * m.head_dim * (m.v_dim + 1)
            elif isinstance(m, DifferentialAttentionSpec):
                seen = sum(p + 1 if m.window is None else min(p + 1, m.window + min(m.keep_first, max(0, p + 1 - m.window)))
                           for p in range(tokens))
                flops += 2.0 * seen * 2 * m.n_heads * (m.head_dim + m.v_dim)
            else:
                flops += 2.0 * (tokens * (tokens + 1) / 2) * m.n_heads * (m.head_dim + m.v_dim)
        return flops
