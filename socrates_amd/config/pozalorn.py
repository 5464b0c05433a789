"""Typed configuration of Pozalorn (``"architecture": "Pozalorn"``).

A decoder whose layers differ: ``layers`` lists them, each with the ``type`` of its mixer (``gla``:
gated linear attention with a decay per key channel that depends on the token; ``attention``:
grouped-query softmax attention over a sliding window and, before it, one mean key and value per
block of tokens, with q and k normed over the whole projection and values turned by position;
``parallel``: windowed softmax attention with a learned sink per head beside lightning attention,
their results scaled and added), the mixer's sizes, and its feed-forward (``dense``: gated with the
tanh form of gelu; or none). A sublayer reads the stream itself and its result is RMS-normed before
it is added; after every layer the stream is replaced by a stored weighting of the embedding output
and all layers' results so far. Tensor names: layer i's start with ``l<i>.``, the mixer's with
``l<i>.mix.`` (``.left.`` / ``.right.`` in a parallel mixer), the feed-forward's with ``l<i>.mlp.``.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Tuple

from .mitisun import _freeze, _positive_int, _thaw
from .qwen3 import ConfigError
from .specs import (BlockSpec, DepthAverageSpec, GatedLinearAttentionSpec, GeluGLUSpec, LightningAttentionSpec, ModelPlan,
                    PairRopeSpec, ParallelMixerSpec, RMSNormSpec, RunStep, WindowAttentionSpec)
from .tedulorn import _number

_NAMES = (("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("ffn", "mlp"), ("depth", "dwa"))
_ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "rot", "mask")
_MIXER_KEYS = {
    "gla": ("heads", "dim", "vdim", "tau"),
    "attention": _ATTENTION_KEYS,
    "parallel": ("left", "right", "left_scale", "right_scale"),
}
_LIGHTNING_KEYS = ("heads", "dim", "vdim", "decay")


def _ints(where, m, keys):
    for k in keys:
        _positive_int(where, k, m[k])


def _lacking(where, m, keys):
    if not isinstance(m, dict):
        raise ConfigError(f"{where}: no mixer sizes")
    lacking = [k for k in keys if k not in m]
    if lacking:
        raise ConfigError(f"{where}: mixer lacks {lacking}")


def _check_attention(where, m, pooled):
    _lacking(where, m, _ATTENTION_KEYS)
    _ints(where, m, ("heads", "kv_heads", "dim", "vdim"))
    _number(where, "scale", m["scale"])
    if m["heads"] % m["kv_heads"]:
        raise ConfigError(f"{where}: {m['heads']} heads do not divide into {m['kv_heads']} kv heads")
    rot = m["rot"]
    if rot is not None:
        if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
            raise ConfigError(f"{where}: rot needs base and dims")
        dims = rot["dims"]
        if not isinstance(dims, int) or isinstance(dims, bool) or dims < 0 or dims % 2 or dims > m["dim"]:
            raise ConfigError(f"{where}: rot.dims must be even and at most the head size {m['dim']}, found {dims!r}")
        _number(where, "rot.base", rot["base"])
        sc = rot.get("scaling")
        if sc is not None:
            for k in ("factor", "low", "high", "original"):
                if not isinstance(sc, dict) or k not in sc:
                    raise ConfigError(f"{where}: rot.scaling needs factor, low, high and original")
                _number(where, f"rot.scaling.{k}", sc[k])
            if not sc["high"] > sc["low"]:
                raise ConfigError(f"{where}: rot.scaling.high must lie above rot.scaling.low")
    mask = m["mask"]
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"{where}: mask needs size")
        _positive_int(where, "mask.size", mask.get("size"))
        if mask.get("pool") is not None:
            _positive_int(where, "mask.pool", mask["pool"])
    if pooled:
        if rot is None or m["vdim"] % 2:
            raise ConfigError(f"{where}: values turned by position need rot.base and an even vdim")


def _check_lightning(where, m):
    _lacking(where, m, _LIGHTNING_KEYS)
    _ints(where, m, ("heads", "dim", "vdim"))
    decay = m["decay"]
    if not isinstance(decay, (list, tuple)) or len(decay) != m["heads"]:
        raise ConfigError(f"{where}: decay lists one number per head ({m['heads']})")
    for x in decay:
        _number(where, "decay", x, positive=False)


@dataclass(frozen=True)
class PozalornConfig:
    vocab: int
    width: int
    layers: Tuple[tuple, ...]         # as config.json lists them (validated, frozen)
    norm_eps: float
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Pozalorn"

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "PozalornConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing} (required for Pozalorn)")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["norm"], dict) or not d["norm"].get("eps", 0) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("layers must list at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            where = f"layer {i}"
            kind = layer.get("type")
            if kind not in _MIXER_KEYS:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {sorted(_MIXER_KEYS)}")
            m = layer.get("mixer")
            _lacking(where, m, _MIXER_KEYS[kind])
            if kind == "gla":
                _ints(where, m, ("heads", "dim", "vdim"))
                _number(where, "tau", m["tau"])
            elif kind == "attention":
                _check_attention(where, m, pooled=True)
            else:
                _check_attention(where + " (left)", m["left"], pooled=False)
                _check_lightning(where + " (right)", m["right"])
                _number(where, "left_scale", m["left_scale"], positive=False)
                _number(where, "right_scale", m["right_scale"], positive=False)
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}: feed-forward kind {mlp.get('kind')!r} is not known (dense)")
                _positive_int(where, "mlp.ff", mlp.get("ff"))
            layers.append(json.loads(json.dumps(layer)))       # a copy of plain values
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(vocab=d["vocab"], width=d["width"], layers=tuple(_freeze(x) for x in layers),
                   norm_eps=float(d["norm"]["eps"]), eos_token_ids=eos_ids, architecture=d.get("architecture", "Pozalorn"))

    @classmethod
    def from_json(cls, path) -> "PozalornConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    # ---- writing -----------------------------------------------------------------
    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "layers": [_thaw(x) for x in self.layers],
               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ---- the layer recipe -------------------------------------------------------------
    def _attention(self, m, pooled):
        rot, mask = m["rot"], m["mask"]
        position = None
        if rot is not None and rot["dims"]:
            sc = rot.get("scaling")
            stretch = None if sc is None else tuple(float(sc[k]) for k in ("factor", "low", "high", "original"))
            position = PairRopeSpec(dims=rot["dims"], base=float(rot["base"]), stretch=stretch)
        return WindowAttentionSpec(
            hidden=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"], v_dim=m["vdim"],
            scale=float(m["scale"]), eps=self.norm_eps, qk_norm="whole" if pooled else "head", position=position,
            window=None if mask is None else mask["size"],
            pool=0 if mask is None or not pooled else int(mask.get("pool") or 0),
            sinks=not pooled, qkv_bias=True, o_bias=not pooled, value_base=float(rot["base"]) if pooled else None)

    def _mixer(self, layer):
        d, eps = self.width, self.norm_eps
        m = layer["mixer"]
        if layer["type"] == "gla":
            return GatedLinearAttentionSpec(hidden=d, n_heads=m["heads"], head_dim=m["dim"], v_dim=m["vdim"],
                                            tau=float(m["tau"]), eps=eps)
        if layer["type"] == "attention":
            return self._attention(m, pooled=True)
        r = m["right"]
        right = LightningAttentionSpec(hidden=d, n_heads=r["heads"], head_dim=r["dim"], v_dim=r["vdim"],
                                       decays=tuple(float(x) for x in r["decay"]), eps=eps)
        return ParallelMixerSpec(left=self._attention(m["left"], pooled=False), right=right,
                                 left_scale=float(m["left_scale"]), right_scale=float(m["right_scale"]))

    def plan(self) -> ModelPlan:
        d, eps = self.width, self.norm_eps
        layers = [_thaw(x) for x in self.layers]
        norm = RMSNormSpec(d, eps, tensor="")
        blocks, ignorable = [], []
        for i, layer in enumerate(layers):
            mlp = layer.get("mlp")
            ffn = None if mlp is None else GeluGLUSpec(d, mlp["ff"])
            blocks.append(BlockSpec(mixer=self._mixer(layer), ffn=ffn, norm1=norm, norm2=None if ffn is None else norm,
                                    prefix=f"l{i}.", names=_NAMES, arrangement="postnorm_depth",
                                    depth=DepthAverageSpec(index=i, n_layers=len(layers))))
            if ffn is None:
                ignorable.append(f"l{i}.norm2")
        return ModelPlan(
            architecture=self.architecture, vocab_size=self.vocab, hidden=d, layers=tuple(blocks),
            order=tuple(RunStep(layer=i, cache=i) for i in range(len(blocks))), final_norm=norm,
            embedding_name="embed", final_norm_prefix="final.norm", head_name="head",
            eos_token_ids=self.eos_token_ids, ignorable=tuple(ignorable))

    # ---- byte and flop counts ---------------------------------------------------------
    def _matrices(self):
        from ..parts import expected_tensors
        return {name: decl for name, decl in expected_tensors(self.plan()).items()
                if decl.kind == "matrix" and len(decl.shape) == 2 and name != "embed"}

    def step_weight_bytes(self, batch: int, item: int) -> int:
        """Bytes of weights that a decode step reads (every matrix once, the embedding's rows aside)."""
        return int(sum(max(decl.shape[0], 1) * max(decl.shape[1], 1) for decl in self._matrices().values()) * item)

    @staticmethod
    def _mixers_of(block):
        m = block.mixer
        return (m.left, m.right) if isinstance(m, ParallelMixerSpec) else (m,)

    def step_cache_bytes(self, batch: int, context: int, item: int) -> int:
        """Bytes of cache and state that a decode step of ``batch`` requests behind ``context`` tokens reads."""
        total = 0
        for block in self.plan().layers:
            for m in self._mixers_of(block):
                if isinstance(m, WindowAttentionSpec):
                    seen = context if m.window is None else min(context, m.window)
                    if m.pool:
                        seen += max(0, context - m.window) // m.pool
                    total += item * 2 * m.n_kv_heads * m.cache_width * seen
                else:
                    total += 4 * m.n_heads * m.head_dim * m.v_dim
        return batch * total

    def prefill_flops(self, tokens: int) -> float:
        """Multiply-adds times two of one prompt of ``tokens`` tokens from position 0: every matrix (the head at
        one position), attention scores and sums over what each token sees, and the recurrences (per token and
        head, state size times four)."""
        flops = 0.0
        for name, decl in self._matrices().items():
            flops += 2.0 * (1 if name == "head" else tokens) * max(decl.shape[0], 1) * max(decl.shape[1], 1)
        for block in self.plan().layers:
            for m in self._mixers_of(block):
                if isinstance(m, WindowAttentionSpec):
                    seen = 0
                    for p in range(tokens):
                        n = p + 1 if m.window is None else min(p + 1, m.window)
                        if m.pool:
                            n += max(0, p - m.window + 1) // m.pool
                        seen += n
                    flops += 2.0 * seen * m.n_heads * (m.head_dim + m.v_dim)
                else:
                    flops += 4.0 * tokens * m.n_heads * m.head_dim * m.v_dim
        return flops
