"""Architecture-neutral description of a decoder: part specs and the model plan.

A *spec* is a frozen dataclass holding every size and constant one part needs.
A *plan* lists the specs of all layers, the order in which layers run, and the
tensor name each parameter has on disk. An architecture's configuration class
(for example ``Qwen3Config``) produces a plan; nothing below the plan knows
which architecture it came from.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x / sqrt(mean(x^2) + eps) * w  over the last ``dim`` elements. ``tensor``: the local
    name of w on disk ("": the tensor carries the norm's own name)."""
    dim: int
    eps: float
    tensor: str = "weight"


@dataclass(frozen=True)
class RopeSpec:
    """Rotate-half rotary encoding over the first ``rotary_dim`` of each head.

    inv_freq[j] = theta ** (-2j / rotary_dim) / factor, pairs are (j, j + rotary_dim/2).
    ``factor`` (1: none; the reference's model has none) stretches the positions a checkpoint was
    trained on by that much (linear position interpolation).
    """
    head_dim: int
    theta: float
    rotary_dim: int = 0          # 0 means the whole head
    factor: float = 1.0

    def __post_init__(self):
        if self.rotary_dim == 0:
            object.__setattr__(self, "rotary_dim", self.head_dim)
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and <= head_dim {self.head_dim}")
        if not self.factor > 0:
            raise ValueError("factor must be positive")


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache.

    ``window`` = None: a query at position p sees keys 0..p. ``window`` = w: it
    sees keys max(0, p-w+1)..p. ``qk_norm`` is applied per head before
    ``position``; either may be None. Terms that other architectures add to the
    scores, all off by default: ``distance_slopes`` (one per query head: slope *
    (key position - query position) is added to the scaled score), ``softcap`` (the
    score becomes softcap * tanh(score / softcap)), ``sinks`` (a stored tensor
    ``sinks`` [n_heads]: one more logit per head that takes part in the softmax's
    sum and has no value).
    """
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float
    qk_norm: Optional[RMSNormSpec] = None
    position: Optional[object] = None
    window: Optional[int] = None
    softcap: Optional[float] = None
    sinks: bool = False
    distance_slopes: Optional[Tuple[float, ...]] = None

    def __post_init__(self):
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError("softcap must be positive")
        if self.distance_slopes is not None and len(self.distance_slopes) != self.n_heads:
            raise ValueError(f"distance_slopes: one per query head ({self.n_heads}), not {len(self.distance_slopes)}")
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.n_kv_heads}")
        if self.head_dim % 16 or not 16 <= self.head_dim <= 256:
            raise ValueError(f"head_dim {self.head_dim}: the attention kernels take multiples of 16 from 16 to 256")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")


@dataclass(frozen=True)
class SwiGLUSpec:
    """y = Wd((Wu x) * silu(Wg x)), no bias. ``names``: the local names of Wg, Wu and Wd on disk."""
    hidden: int
    intermediate: int
    names: Tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")


@dataclass(frozen=True)
class ScalarRMSNormSpec:
    """y = x / sqrt(mean(x^2) + eps) * g over the last ``dim`` elements, with one stored
    number g for all of them (the tensor carries the norm's own name, no suffix)."""
    dim: int
    eps: float


@dataclass(frozen=True)
class PairRopeSpec:
    """Rotary encoding in the interleaved layout: elements 2i and 2i + 1 of the first ``dims``
    of a vector are one pair, turned by position * base ** (-2i / dims); the rest passes."""
    dims: int
    base: float
    # (factor, low, high, original): a frequency whose wavelength is longer than original / low is divided
    # by factor, one whose wavelength is shorter than original / high stays, and between the two, with
    # s = (original / wavelength - low) / (high - low), it becomes (1 - s) f / factor + s f. None: no stretch.
    stretch: Optional[Tuple[float, float, float, float]] = None
    # (factor, original, fast, slow): the stretch as a linear ramp over the pair index. With
    # index(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(index(fast)), 0) and
    # hi = min(ceil(index(slow)), dims - 1), pair i has r = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) and the
    # frequency r f / factor + (1 - r) f; cosines and sines are multiplied by 0.1 ln(factor) + 1 (``magnitude``).
    ramp: Optional[Tuple[float, float, float, float]] = None

    def __post_init__(self):
        if self.stretch is not None and self.ramp is not None:
            raise ValueError("a rotation is stretched by wavelength or by a ramp over the pair index, not both")
        if self.ramp is not None:
            factor, original, fast, slow = self.ramp
            if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and self.base > 1):
                raise ValueError(f"ramp (factor, original, fast, slow) = {self.ramp}: all positive, over a base above 1")
        if self.dims < 2 or self.dims % 2:
            raise ValueError(f"a rotation over pairs needs an even number of dimensions, not {self.dims}")
        if not self.base > 0:
            raise ValueError("the rotation's base must be positive")
        if self.stretch is not None:
            factor, low, high, original = self.stretch
            if not (factor > 0 and original > 0 and high > low > 0):
                raise ValueError(f"stretch (factor, low, high, original) = {self.stretch}: factor and original are "
                                 "positive and high lies above low")

    def frequencies(self):
        """The dims / 2 frequencies as Python floats (double precision)."""
        import math
        out = []
        for i in range(self.dims // 2):
            f = self.base ** (-2.0 * i / self.dims)
            if self.stretch is not None:
                factor, low, high, original = self.stretch
                wave = 2.0 * math.pi / f
                if wave > original / low:
                    f = f / factor
                elif wave >= original / high:
                    t = (original / wave - low) / (high - low)
                    f = (1.0 - t) * f / factor + t * f
            out.append(f)
        if self.ramp is not None:
            factor, original, fast, slow = self.ramp

            def index(turns):
                return self.dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))
            lo = max(math.floor(index(fast)), 0)
            hi = min(math.ceil(index(slow)), self.dims - 1)
            for i, f in enumerate(out):
                r = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
                out[i] = r * f / factor + (1.0 - r) * f
        return out

    @property
    def magnitude(self) -> float:
        """What cosines and sines are multiplied by (1 without a ramp)."""
        import math
        return 1.0 if self.ramp is None else 0.1 * math.log(self.ramp[0]) + 1.0


@dataclass(frozen=True)
class ClampedGLUSpec:
    """y = Wd(g * sigmoid(slope * g) * (u + 1)) with g = min(Wg x, limit) and
    u = clamp(Wu x, -limit, limit), no bias."""
    hidden: int
    intermediate: int
    limit: float
    slope: float = 1.702

    def __post_init__(self):
        if not self.limit > 0:
            raise ValueError("limit must be positive")


@dataclass(frozen=True)
class SigmoidGateSpec:
    """sigmoid(W h + b), [dim] from [dim]: what a block multiplies a branch's result by."""
    dim: int


@dataclass(frozen=True)
class WkvSpec:
    """Time mixing with a matrix state per head and a decay per key channel that depends on
    the token: each of r, k, v, g, w reads its own blend of the token's input and the one
    before it; o_t = (S + diag(u) k_t v_t^T)^T r_t, S <- diag(w_t) S + k_t v_t^T with
    w = exp(-exp(W2 tanh(W1 x_w) + w0)); each head's o over its root mean square, times a gain,
    times silu(g), then the output projection. ``decay_rank`` 0: whatever W1 holds on disk."""
    hidden: int
    n_heads: int
    head_dim: int
    eps: float
    decay_rank: int = 0

    def __post_init__(self):
        if self.n_heads < 1 or not 1 <= self.head_dim <= 256:
            raise ValueError(f"wkv: {self.n_heads} heads of {self.head_dim}: head sizes run from 1 to 256")


@dataclass(frozen=True)
class Mamba2Spec:
    """State-space mixing with a scalar decay per head (Mamba-2): the input projection gives
    [z | x | B | C | dt]; x, B, C pass a causal convolution of ``conv_taps`` taps per channel
    and silu; dt = softplus(dt + bias); S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x
    per head (``state`` x ``head_dim``), heads sharing B and C in ``n_groups`` groups; y times
    silu(z), RMS-normed in ``norm_groups`` equal parts, times a gain, then the output projection."""
    hidden: int
    n_heads: int
    head_dim: int
    state: int
    n_groups: int
    conv_taps: int
    norm_groups: int
    eps: float

    def __post_init__(self):
        if self.n_heads % self.n_groups:
            raise ValueError(f"mamba2: {self.n_heads} heads do not divide into {self.n_groups} groups")
        if (self.n_heads * self.head_dim) % self.norm_groups:
            raise ValueError(f"mamba2: {self.n_heads * self.head_dim} channels do not divide into {self.norm_groups} norm groups")
        if not 1 <= self.state <= 256 or self.head_dim < 1 or self.conv_taps < 1:
            raise ValueError(f"mamba2: state {self.state} (1 to 256), head size {self.head_dim}, {self.conv_taps} taps")

    @property
    def inner(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.n_groups * self.state


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are expanded from one cached latent per token.

    Queries: q = Wuq rmsnorm(Wdq h), per head [``head_dim`` plain | ``rot_dim`` rotated].
    Keys and values: Wdkv h = [latent (``kv_rank``, RMS-normed) | one rotated key part
    (``rot_dim``) that all heads share]; per head the plain key is Wuk latent, the value Wuv
    latent (``v_dim``). score = scale * (q_plain . k_plain + q_rot . k_rot); a query at
    position p sees keys p - window + 1 .. p (all up to p if ``window`` is None).
    ``own_kv`` False: the layer has no Wdkv and reads the cache slot another layer writes.
    ``keep``: how many positions back the cache slot has to hold (the widest window of all
    layers that read it; None: all)."""
    hidden: int
    n_heads: int
    head_dim: int
    rot_dim: int
    v_dim: int
    kv_rank: int
    q_rank: int
    scale: float
    position: PairRopeSpec
    eps: float
    window: Optional[int] = None
    keep: Optional[int] = None
    own_kv: bool = True

    def __post_init__(self):
        if self.position.dims > self.rot_dim:
            raise ValueError(f"the rotation covers {self.position.dims} dimensions, the rotated part has {self.rot_dim}")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")
        if self.window is None and self.keep is not None or (
                self.window is not None and self.keep is not None and self.keep < self.window):
            raise ValueError("the cache must keep at least the layer's own window")
        if not 16 <= self.cache_width <= 256:
            raise ValueError(f"latent of {self.kv_rank} + rotated part of {self.rot_dim}: the attention kernels take "
                             "up to 256 together")

    @property
    def cache_width(self) -> int:
        """Elements per cached token: latent and rotated key part, padded to the kernels' step."""
        return (self.kv_rank + self.rot_dim + 15) // 16 * 16


@dataclass(frozen=True)
class GatedWindowAttentionSpec:
    """Grouped-query softmax attention whose keys and values may differ in size, over a window that
    keeps the first tokens visible, with a gate per head.

    q, k [heads x ``head_dim``], v [kv heads x ``v_dim``]; q and k RMS-normed per head with one gain
    each (``qk_norm_eps`` None: no norm), then turned by ``position``. A query at position p sees key
    j <= p if p - j < ``window`` or j < ``keep_first`` (``window`` None: all). ``sink`` adds one weight of
    score 0 and no value to the softmax's sum: p_j = exp(s_j) / (1 + sum exp(s_j)). ``value_blend``
    "first": the layer's values are what later layers blend with; "later": its values become
    (1 - l) v + l v_first, with l the stored number ``vmix`` and v_first the "first" layer's values of
    the same token (the blend is what the cache holds); None: no blend. ``head_gate``: head h's result
    is multiplied by sigmoid(W_g x)_h before the output projection."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_dim: int
    scale: float
    qk_norm_eps: Optional[float] = None
    position: Optional[object] = None
    window: Optional[int] = None
    keep_first: int = 0
    sink: bool = False
    value_blend: Optional[str] = None
    stores_blend: bool = False           # the file holds ``vmix`` also where the layer does not use it
    head_gate: bool = False

    def __post_init__(self):
        if self.n_heads < 1 or self.n_kv_heads < 1 or self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.n_kv_heads}")
        if not 1 <= self.head_dim <= 256 or not 1 <= self.v_dim <= 256:
            raise ValueError(f"head sizes {self.head_dim} and {self.v_dim}: the attention kernels take up to 256")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")
        if self.keep_first < 0:
            raise ValueError("keep_first is not negative")
        if self.value_blend not in (None, "first", "later"):
            raise ValueError(f"value_blend {self.value_blend!r}: first, later or None")
        if not self.scale > 0:
            raise ValueError("scale must be positive")

    @property
    def cache_width(self) -> int:
        """Elements per cached key and per cached value: the larger of the two sizes, padded to the
        kernels' step."""
        return (max(self.head_dim, self.v_dim) + 15) // 16 * 16


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head and no softmax or denominator: q, k [heads x
    ``head_dim``] turned by ``position``, k scaled by head_dim^-1/2 after it, v [heads x ``v_dim``];
    S <- decay_h S + k v^T, o = S^T q per head; each head's o over its root mean square (eps, no gain),
    times silu(W_g x), then the output projection. The state is float32 and starts at zero."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    decays: Tuple[float, ...]
    eps: float
    position: Optional[object] = None

    def __post_init__(self):
        if self.n_heads < 1 or len(self.decays) != self.n_heads:
            raise ValueError(f"retention: {len(self.decays)} decays for {self.n_heads} heads")
        if not 1 <= self.head_dim <= 256 or self.v_dim < 1:
            raise ValueError(f"retention: heads of {self.head_dim} (1 to 256) and {self.v_dim}")


@dataclass(frozen=True)
class ReluSquaredSpec:
    """y = Wd(relu(Wu x)^2), no bias."""
    hidden: int
    intermediate: int


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A mixture of ``n_experts`` clamped gated feed-forwards (``expert``) of which a token uses ``top``.

    Scores s = softmax(W_router x) in float32; the choice goes by s + ``correction`` (a stored vector;
    ``corrected`` False: by s). Experts form ``n_groups`` equal groups of neighbours; a group's score is
    its largest choice score, and only experts of the ``keep_groups`` best groups can be chosen. The
    weights are the chosen experts' s over their sum (+ ``renorm_eps``). ``shared``: one more such
    feed-forward that every token uses, added unweighted (None: none).

    ``scoring`` "sigmoid": s = sigmoid(W_router x) in place of the softmax. ``group_top`` = n: a group's score is the
    sum of its n largest choice scores (1: its largest). ``scale``: the weights are multiplied by it. ``expert`` and
    ``shared`` may also be a ``SwiGLUSpec`` (a plain silu gate, no clamp). ``shared_gate``: the shared expert's
    result is multiplied by sigmoid(w_sg . x), one number per token (stored as ``shared.sg`` [1, hidden])."""
    hidden: int
    n_experts: int
    top: int
    expert: object
    n_groups: int = 1
    keep_groups: int = 1
    shared: object = None
    corrected: bool = True
    renorm_eps: float = 1e-20
    scoring: str = "softmax"
    group_top: int = 1
    scale: float = 1.0
    shared_gate: bool = False

    def __post_init__(self):
        if self.scoring not in ("softmax", "sigmoid"):
            raise ValueError(f"scoring {self.scoring!r}: softmax or sigmoid")
        if self.group_top < 1:
            raise ValueError("a group's score sums at least its largest score")
        if self.shared_gate and self.shared is None:
            raise ValueError("a gate on the shared expert needs a shared expert")
        if not 1 <= self.top <= self.n_experts:
            raise ValueError(f"a token uses {self.top} of {self.n_experts} experts")
        if self.n_groups < 1 or self.n_experts % self.n_groups or not 1 <= self.keep_groups <= self.n_groups:
            raise ValueError(f"{self.n_experts} experts in {self.n_groups} groups, {self.keep_groups} kept")
        if self.keep_groups * (self.n_experts // self.n_groups) < self.top:
            raise ValueError(f"{self.keep_groups} groups of {self.n_experts // self.n_groups} experts hold fewer than {self.top}")


@dataclass(frozen=True)
class TokenSideSpec:
    """A per-layer input that depends on the token alone: with e the layer's ``dim`` columns (from
    ``index`` * dim on) of a table [vocab, ``n_layers`` * dim] that all layers share (``table_name``, a name
    of the whole model), y = W_proj(gelu_tanh(W_gate x) * e) and x <- x + y / rms(y) * gain."""
    hidden: int
    dim: int
    index: int
    n_layers: int
    vocab: int
    eps: float
    table_name: str = "side.embed"


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Grouped-query softmax attention over a sliding window, with what designs put around it.

    q, k [heads x ``head_dim``], v [kv heads x ``v_dim``], each with a bias if ``qkv_bias``. ``qk_norm``:
    "head" (RMS norm over each head, one gain of head_dim for all heads), "whole" (RMS norm over the whole
    projection of q, and of k, with a gain of that size) or None. ``position`` turns interleaved pairs of
    q and k. ``value_base`` = B: the value of position j is turned by j over pairs (2m, 2m + 1) of all v_dim
    elements with the frequencies B^(-2m / v_dim), and cached so; a head's result at position i is turned
    back by i (None: values as they are). A query at position i sees key j with
    0 <= i - j < ``window`` (None: all j <= i) and, with ``pool`` = P > 0, one mean key and mean value (of
    what the cache holds) for every block bP .. bP + P - 1 with bP + P - 1 <= i - window, in the same
    softmax. ``sinks``: a stored number per head whose exponential joins the softmax's denominator.

    ``qk_norm`` "turned": q and k are divided by their root mean square per head after the rotation, with no gain.
    ``tied_values``: there is no value projection; a token's values are its keys as projected, before norm and
    rotation (v_dim equals head_dim). ``softcap`` = c: a scaled score s becomes c tanh(s / c). ``head_gate``: head
    h's result is multiplied by sigmoid(W_g x)_h (stored as ``g`` [heads, hidden]) before the output projection.
    ``keep_first``: with a window, the keys at positions below it stay visible to every later token."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_dim: int
    scale: float
    eps: float
    qk_norm: Optional[str] = None
    position: Optional[PairRopeSpec] = None
    window: Optional[int] = None
    pool: int = 0
    sinks: bool = False
    qkv_bias: bool = False
    o_bias: bool = False
    value_base: Optional[float] = None
    tied_values: bool = False
    softcap: Optional[float] = None
    head_gate: bool = False
    keep_first: int = 0

    def __post_init__(self):
        if self.n_heads < 1 or self.n_kv_heads < 1 or self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.n_kv_heads}")
        if not 1 <= self.head_dim <= 256 or not 1 <= self.v_dim <= 256:
            raise ValueError(f"head sizes {self.head_dim} and {self.v_dim}: the attention kernels take up to 256")
        if self.qk_norm not in (None, "head", "whole", "turned"):
            raise ValueError(f"qk_norm {self.qk_norm!r}: head, whole, turned or None")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")
        if self.tied_values and (self.v_dim != self.head_dim or self.value_base is not None):
            raise ValueError("values that are the keys have the keys' size and are not turned")
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError("softcap must be positive")
        if self.keep_first < 0 or (self.keep_first and self.pool):
            raise ValueError("keep_first is not negative, and not combined with pooled blocks")
        if self.pool < 0 or (self.pool and self.window is None):
            raise ValueError("pooled blocks lie before a window: pool needs a window and is not negative")
        if self.position is not None and self.position.dims > self.head_dim:
            raise ValueError(f"the rotation covers {self.position.dims} dimensions, a head has {self.head_dim}")
        if self.value_base is not None and (not self.value_base > 0 or self.v_dim % 2):
            raise ValueError("turned values need a positive base and an even v_dim")
        if not self.scale > 0:
            raise ValueError("scale must be positive")

    @property
    def cache_width(self) -> int:
        """Elements per cached key and per cached value: the larger of the two sizes, padded to the
        kernels' step."""
        return (max(self.head_dim, self.v_dim) + 15) // 16 * 16


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Grouped-query attention with two softmax maps per head over the same values, the second subtracted.

    q holds, head by head, [map 1 | map 2] of ``head_dim`` each, k likewise per kv head; v [kv heads x ``v_dim``];
    all three and the output projection with biases. ``position`` turns interleaved pairs of every map of q and k.
    Query i sees key j <= i if i - j < ``window`` or j < ``keep_first`` (``window`` None: all). With a1, a2 the two
    maps' results and lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff`` (four stored vectors of head_dim), a head's
    result is (a1 - lambda a2) over its root mean square (eps inside the root, no gain) times (1 - diff).
    ``own_kv`` False: the layer has no k and v projections and reads the cache slot another such layer writes.
    ``cache_window`` / ``cache_keep_first``: what the cache slot has to hold, the widest of all layers that read it
    (``cache_window`` 0: this layer's own window and kept keys; None: every position)."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_dim: int
    scale: float
    eps: float
    diff: float
    position: Optional[PairRopeSpec] = None
    window: Optional[int] = None
    keep_first: int = 0
    own_kv: bool = True
    cache_window: Optional[int] = 0
    cache_keep_first: int = 0

    @property
    def cache_mask(self):
        """(window, kept first keys) of what the cache slot holds."""
        if self.cache_window == 0:
            return self.window, (self.keep_first if self.window is not None else 0)
        return self.cache_window, (self.cache_keep_first if self.cache_window is not None else 0)

    def __post_init__(self):
        if self.n_heads < 1 or self.n_kv_heads < 1 or self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.n_kv_heads}")
        if not 1 <= self.head_dim <= 256 or not 1 <= self.v_dim <= 256:
            raise ValueError(f"head sizes {self.head_dim} and {self.v_dim}: the attention kernels take up to 256")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")
        if self.keep_first < 0 or self.cache_keep_first < 0 or (self.cache_window is not None and self.cache_window < 0):
            raise ValueError("keep_first and cache_window are not negative")
        if self.position is not None and self.position.dims > self.head_dim:
            raise ValueError(f"the rotation covers {self.position.dims} dimensions, a map has {self.head_dim}")
        if not self.scale > 0:
            raise ValueError("scale must be positive")
        if self.window is None:
            if self.cache_window:
                raise ValueError("the cache must keep every position for a layer without a window")
        elif self.cache_window and (self.cache_window < self.window or
                                    (self.keep_first and self.cache_keep_first < self.keep_first)):
            raise ValueError("the cache must keep at least the layer's own window and first keys")

    @property
    def cache_width(self) -> int:
        """Elements per cached key and per cached value: the larger of the two sizes, padded to the
        kernels' step."""
        return (max(self.head_dim, self.v_dim) + 15) // 16 * 16


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A matrix memory per head with exponential gates (mLSTM). q = Wq h * head_dim^-1/2, k = Wk h, v = Wv h; per
    head a log input gate i = cap tanh((Wi h + bi) / cap) and a log forget gate f = logsigmoid(cap tanh((Wf h + bf) /
    cap)); with a running maximum m (0 at the start): m' = max(f + m, i), S <- exp(f + m - m') S + exp(i - m') k v^T,
    n likewise with k alone, o = S^T q / (max(|n . q|, exp(-m')) + ``den_eps``). Each head's o over its root mean
    square (eps, no gain of its own), the heads together times a gain and sigmoid(Wg h), then the output projection.
    S, n and m are float32 and start at zero."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    gate_cap: float
    eps: float
    den_eps: float = 1e-6

    def __post_init__(self):
        if self.n_heads < 1 or not 1 <= self.head_dim <= 256 or self.v_dim < 1:
            raise ValueError(f"matrix memory: {self.n_heads} heads of {self.head_dim} (1 to 256) and {self.v_dim}")
        if not self.gate_cap > 0:
            raise ValueError("gate_cap must be positive")


@dataclass(frozen=True)
class GatedLinearAttentionSpec:
    """Linear attention with a decay per key channel that depends on the token: q = Wq h * head_dim^-1/2,
    k = Wk h, v = Wv h; alpha = sigmoid(Wa2 (Wa1 h) + b)^(1 / tau) [heads x head_dim];
    S <- diag(alpha) S + k v^T, o = S^T q per head; each head's o RMS-normed with one gain of v_dim for
    all heads, times silu(Wg h), then the output projection. The state is float32 and starts at zero.
    ``decay_rank`` 0: whatever Wa1 holds on disk."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    tau: float
    eps: float
    decay_rank: int = 0

    def __post_init__(self):
        if self.n_heads < 1 or not 1 <= self.head_dim <= 256 or self.v_dim < 1:
            raise ValueError(f"gated linear attention: {self.n_heads} heads of {self.head_dim} (1 to 256) and {self.v_dim}")
        if not self.tau > 0:
            raise ValueError("tau must be positive")


@dataclass(frozen=True)
class LightningAttentionSpec:
    """Linear attention with a fixed decay per head over activated projections: q = silu(Wq h),
    k = silu(Wk h), v = silu(Wv h); S <- decay_h S + k v^T, o = S^T q; the heads together RMS-normed with
    a gain, times sigmoid(Wg h), then the output projection. The state is float32 and starts at zero."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    decays: Tuple[float, ...]
    eps: float

    def __post_init__(self):
        if self.n_heads < 1 or len(self.decays) != self.n_heads:
            raise ValueError(f"lightning attention: {len(self.decays)} decays for {self.n_heads} heads")
        if not 1 <= self.head_dim <= 256 or self.v_dim < 1:
            raise ValueError(f"lightning attention: heads of {self.head_dim} (1 to 256) and {self.v_dim}")


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side on the same input: ``left_scale`` * left(h) + ``right_scale`` * right(h);
    their tensors lie under ``left.`` and ``right.``, and each keeps its own cache or state."""
    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass(frozen=True)
class GeluGLUSpec:
    """y = Wd(gelu_tanh(Wg x) * (Wu x)), no bias;
    gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""
    hidden: int
    intermediate: int


@dataclass(frozen=True)
class DepthAverageSpec:
    """What goes on from layer ``index``: sum over j = 0 .. index + 1 of w[j] X_j, with X_0 the embedding
    output, X_(j+1) layer j's own result (before this sum) and w a stored vector of index + 2 numbers.
    ``n_layers``: how many layers the model has (a step keeps that many results and one)."""
    index: int
    n_layers: int


@dataclass(frozen=True)
class BlockSpec:
    """One layer: which mixer, feed-forward and norms, how they are arranged,
    and the prefix its tensors carry on disk.

    ``arrangement`` "prenorm": h = x + mixer(norm1(x)); y = h + ffn(norm2(h)).
    ``names`` maps the role of each sub-part to the name segment after
    ``prefix`` (for example {"mixer": "self_attn"}).
    """
    mixer: object
    ffn: object
    norm1: object
    norm2: object
    prefix: str
    names: Tuple[Tuple[str, str], ...] = (
        ("norm1", "input_layernorm"), ("mixer", "self_attn"),
        ("norm2", "post_attention_layernorm"), ("ffn", "mlp"))
    arrangement: str = "prenorm"
    # For the arrangement "sandwich": x <- x + mult * post_norm(gate(h) * branch(h)) with
    # h = norm(x), for the mixer and then for the feed-forward (``ffn`` None: the layer has
    # none, and no norm2, post_norm2 or gate2 either); a gate of None multiplies by one.
    post_norm1: object = None
    post_norm2: object = None
    gate1: object = None
    gate2: object = None
    residual_mult: float = 1.0
    # For the arrangement "prenorm_side": prenorm, then x <- x + side(x) on the stream itself (``side``
    # None: none); ``ffn`` None: the layer has no feed-forward and no norm2.
    side: object = None
    # For the arrangement "postnorm_depth": x <- x + norm1(mixer(x)); x <- x + norm2(ffn(x)) (the parts read
    # the stream itself, the norms act on their results; ``ffn`` None: no feed-forward and no norm2); then
    # what goes on is ``depth``'s weighted sum of the embedding output and all layers' results so far.
    depth: object = None

    ROLES = ("norm1", "mixer", "norm2", "ffn", "post_norm1", "post_norm2", "gate1", "gate2", "side", "depth")

    def name_of(self, role: str) -> str:
        return self.prefix + dict(self.names)[role]


@dataclass(frozen=True)
class RunStep:
    """One entry of the execution order.

    ``layer`` indexes ``ModelPlan.layers`` (a layer may appear more than once);
    ``cache`` is the cache slot this execution uses; ``write`` False means the
    execution only reads what an earlier step wrote into that slot.
    """
    layer: int
    cache: int
    write: bool = True


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[BlockSpec, ...]
    order: Tuple[RunStep, ...]
    final_norm: object
    embedding_name: str
    final_norm_prefix: str
    head_name: Optional[str]      # None: the head is the embedding table (tied)
    eos_token_ids: Tuple[int, ...] = field(default=())
    # (stored name, name of an expected tensor): a checkpoint may also store the first if it
    # holds the very same values as the second (a tied head written out beside the embedding)
    duplicates: Tuple[Tuple[str, str], ...] = field(default=())
    # What some architectures put between the parts (none of it in the reference's model, so
    # the defaults leave the step as it is): the embedding's rows times a constant; the logits
    # times a constant, then logit_softcap * tanh(logits / logit_softcap).
    # names a checkpoint may also hold and that are not read (tensors of a sub-part a layer lacks)
    ignorable: Tuple[str, ...] = field(default=())
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: Optional[float] = None

    def __post_init__(self):
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ValueError("logit_softcap must be positive")
        written = set()
        for step in self.order:
            if not 0 <= step.layer < len(self.layers):
                raise ValueError(f"run step names layer {step.layer}, the plan has {len(self.layers)}")
            if step.write:
                if step.cache in written:
                    raise ValueError(f"cache slot {step.cache} is written by two run steps")
                written.add(step.cache)
            elif step.cache not in written:
                raise ValueError(f"run step reads cache slot {step.cache} before any step wrote it")

    @property
    def n_cache_slots(self) -> int:
        return 1 + max(s.cache for s in self.order) if self.order else 0


def default_order(n_layers: int) -> Tuple[RunStep, ...]:
    """Every layer once, in index order, each with a cache slot of its own."""
    return tuple(RunStep(layer=i, cache=i) for i in range(n_layers))
