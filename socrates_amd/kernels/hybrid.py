"""Wrappers of the kernels in ``csrc/hybrid.hip``: what prepares attention whose keys and values
differ in size and gates its heads, retention, routed experts, the squared-relu activation, a
per-token side input, and the residual sum with a cast. The library is compiled and loaded when
a model first asks for one of them."""

from __future__ import annotations

from ctypes import c_float, c_int, c_longlong

import torch

from .build import load_library
from .common import _HYBRID_SIGNATURES, KernelError, _check, _declare, _ptr

MAX_EXPERTS = 256        # what the routing and sorting kernels hold per token and per workgroup
EXPERT_TILE = 16         # places of one expert that a workgroup of the products per expert takes ...
# ... or, in bfloat16, (tokens per expert on average from which, places). Tiles of 256 places were measured and lost
# (a prompt of 2,048 tokens at 4B-sized layers, 256 tokens per expert on average: 20.5 against 17.6 ms).
EXPERT_TILES_MANY = ((48, 128),)


class ExpertRuns:
    """Tokens sorted by expert: ``place`` [M] (where each (token, choice) pair lies), ``pair_at`` [M] (which
    pair lies at a place), ``offsets`` [E + 1] (each expert's run of places) and ``tiles`` [max_tiles, 2]
    ((expert, first place) of every tile the products walk; expert -1 behind the last)."""
    __slots__ = ("place", "pair_at", "offsets", "tiles", "top", "tile")

    def __init__(self, place, pair_at, offsets, tiles, top, tile):
        self.place, self.pair_at, self.offsets, self.tiles, self.top, self.tile = place, pair_at, offsets, tiles, top, tile


class Hybrid:
    retention_turn_ahead = 16       # tokens of a step's longest portion from which q and k are turned ahead of the walk

    def _hybrid(self):
        lib = getattr(self, "_hybrid_lib", None)
        if lib is None:
            lib = self._hybrid_lib = load_library("hybrid")
            _declare(lib, _HYBRID_SIGNATURES)
        return lib

    def _cols(self, x, name, N, width):
        """``x`` [N, width] in the compute dtype, rows contiguous and apart by at least ``width``."""
        if (x.device.type != "cuda" or x.dtype != self.dtype or tuple(x.shape) != (N, width) or x.stride(1) != 1
                or (N > 1 and x.stride(0) < width)):
            raise KernelError(f"{name}: {tuple(x.shape)} with strides {x.stride()} does not fit [{N}, {width}]")

    # -- attention whose keys and values differ in size ----------------------------------------------------
    def attn_prepare(self, x, cols, Hq, Hkv, D, Dv, P, q_gain, k_gain, eps, inv_freq, rotary_dim, positions,
                     token_rows, slot, first=None, lam=None):
        """x [N, ld] holds, from columns ``cols`` = (q, k, v) on, Hq heads of D, Hkv heads of D and Hkv heads of
        Dv. Queries and keys are RMS-normed per head (gains [D], or None for no norm) and turned over their
        first ``rotary_dim`` elements; values become (1 - lam) v + lam first where ``first`` [N, Hkv * Dv] (it may
        be columns of a wider tensor) and ``lam`` (one float32) are given. Keys and values go to the token's
        place in the pools [pages, Hkv, block, P], zeros behind D and Dv; ``slot`` None: nothing is written.
        Returns q [N, Hq, P], zeros behind D."""
        N, ld = x.shape
        self._want(x, "x", self.dtype)
        col_q, col_k, col_v = cols
        if min(cols) < 0 or col_q + Hq * D > ld or col_k + Hkv * D > ld or col_v + Hkv * Dv > ld:
            raise KernelError(f"queries, keys and values from columns {cols} do not fit rows of {ld}")
        if not (1 <= D <= P and 1 <= Dv <= P and P <= 256) or rotary_dim % 2 or not 0 <= rotary_dim <= D:
            raise KernelError(f"head sizes {D} and {Dv} in pools of {P}, rotation over {rotary_dim}")
        if (q_gain is None) != (k_gain is None):
            raise KernelError("q and k gains come together")
        if q_gain is not None:
            self._want(q_gain, "q gain", torch.float32, (D,))
            self._want(k_gain, "k gain", torch.float32, (D,))
        half = rotary_dim // 2
        if half:
            self._want(inv_freq, "inv_freq", torch.float32, (half,))
        self._want(positions, "positions", torch.int32, (N,))
        self._want(token_rows, "token_rows", torch.int32, (N,))
        ldf = 0
        if first is not None:
            self._cols(first, "the earlier layer's values", N, Hkv * Dv)
            self._want(lam, "blend weight", torch.float32)
            if lam.numel() != 1:
                raise KernelError("the blend weight is one number")
            ldf = first.stride(0)
        n_kv = Hkv
        if slot is None:
            n_kv, kp, vp, table, width, bs = 0, None, None, None, 0, 1
        else:
            self._check_slot(slot, Hkv, P)
            kp, vp, table, width, bs = slot.k, slot.v, slot.block_table, slot.block_table.shape[1], slot.block_size
        q = torch.empty((N, Hq, P), dtype=self.dtype, device=self.device)
        _check(self._hybrid().soc_attn_prepare(
            _ptr(x), c_int(ld), c_int(col_q), c_int(col_k), c_int(col_v), _ptr(first), c_int(ldf), _ptr(lam), _ptr(q),
            _ptr(kp), _ptr(vp), _ptr(table), c_int(width), _ptr(token_rows), _ptr(positions), _ptr(q_gain), _ptr(k_gain),
            _ptr(inv_freq if half else None), c_int(N), c_int(Hq), c_int(n_kv), c_int(D), c_int(Dv), c_int(P), c_int(half),
            c_int(bs), c_float(eps), c_int(self.code), self._stream()), "attn_prepare")
        return q

    def head_gate(self, o, H, P, Dv, gate):
        """o [N, H * P] -> [N, H * Dv]: the first Dv elements of each head times sigmoid(gate[n, h]); ``gate``
        [N, H] may be columns of a wider tensor; None: no gate, the heads' first Dv elements as they are."""
        N = o.shape[0]
        self._want(o, "o", self.dtype, (N, H * P))
        if gate is not None:
            self._cols(gate, "gate logits", N, H)
        if Dv > P:
            raise KernelError(f"{Dv} elements of heads of {P}")
        out = torch.empty((N, H * Dv), dtype=self.dtype, device=self.device)
        _check(self._hybrid().soc_head_gate(_ptr(o), _ptr(gate), c_int(gate.stride(0) if gate is not None else 0), _ptr(out), c_int(N), c_int(H), c_int(P),
                                            c_int(Dv), c_int(self.code), self._stream()), "head_gate")
        return out

    # -- retention ---------------------------------------------------------------------------------------------
    def retention(self, x, cols, H, D, Dv, inv_freq, rotary_dim, k_scale, decays, state, offset, ctx):
        """S <- decay_h S + k v^T, o = S^T q per head over each sequence's tokens, from and into the row's state
        ([H, D, Dv] from ``offset``). x [N, ld] holds q and k (H heads of D) and v (H heads of Dv) from columns
        ``cols`` on; q and k are turned over their first ``rotary_dim`` elements by position and k is scaled by
        ``k_scale``, in float32. float32 [N, H * Dv]."""
        N, ld = x.shape
        self._want(x, "x", self.dtype)
        col_q, col_k, col_v = cols
        if min(cols) < 0 or max(col_q, col_k) + H * D > ld or col_v + H * Dv > ld:
            raise KernelError(f"queries, keys and values from columns {cols} do not fit rows of {ld}")
        if not 1 <= D <= 256 or Dv < 1 or rotary_dim % 2 or not 0 <= rotary_dim <= D:
            raise KernelError(f"retention: heads of {D} and {Dv}, rotation over {rotary_dim}")
        half = rotary_dim // 2
        if half:
            self._want(inv_freq, "inv_freq", torch.float32, (half,))
        self._want(ctx.positions, "positions", torch.int32, (N,))
        self._want(decays, "decays", torch.float32, (H,))
        stride = self._state(state, offset, H * D * Dv, ctx)
        out = torch.empty((N, H * Dv), dtype=torch.float32, device=self.device)
        # a step with a portion of some length: q and k are turned once, ahead of the walk (each of a head's
        # workgroups would turn them again); single tokens and short portions are turned where they are staged
        turned = None
        if half and ctx.max_q_len >= self.retention_turn_ahead:
            turned = torch.empty((N, 2, H * D), dtype=torch.float32, device=self.device)
        _check(self._hybrid().soc_retention(
            _ptr(x), c_int(ld), c_int(col_q), c_int(col_k), c_int(col_v), _ptr(ctx.positions), _ptr(inv_freq if half else None),
            c_int(half), c_float(k_scale), _ptr(decays), c_int(H), c_int(D), c_int(Dv), _ptr(state), stride, c_int(offset),
            _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(turned), c_int(N), _ptr(out), c_int(ctx.n_seqs), c_int(ctx.max_q_len),
            c_int(self.code), self._stream()), "retention")
        return out

    # -- feed-forwards --------------------------------------------------------------------------------------------
    def relu_squared(self, x):
        self._want(x, "x", self.dtype)
        out = torch.empty_like(x)
        _check(self._hybrid().soc_relu_squared(_ptr(x), _ptr(out), c_longlong(x.numel()), c_int(self.code), self._stream()),
               "relu_squared")
        return out

    def moe_route(self, logits, correction, top, n_groups=1, keep_groups=1, renorm_eps=1e-20, scoring="softmax", group_top=1,
                  scale=1.0):
        """logits float32 [N, E] (they may be columns of a wider product): scores are their softmax, or with ``scoring``
        "sigmoid" the sigmoid of each; the choice goes by score + correction among the experts of the ``keep_groups``
        best of ``n_groups`` equal groups of neighbours (a group's score is the sum of its ``group_top`` best choice
        scores). Returns (experts int32 [N, top], weights float32 [N, top]: the chosen scores over their sum, times
        ``scale``)."""
        N, E = logits.shape
        if (logits.device.type != "cuda" or logits.dtype != torch.float32 or logits.stride(1) != 1
                or (N > 1 and logits.stride(0) < E)):
            raise KernelError(f"router logits {tuple(logits.shape)} {logits.dtype} with strides {logits.stride()}")
        if scoring not in ("softmax", "sigmoid") or group_top < 1:
            raise KernelError(f"routing: scoring {scoring!r}, groups scored by their {group_top} best")
        if correction is not None:
            self._want(correction, "correction", torch.float32, (E,))
        if (not 1 <= E <= MAX_EXPERTS or not 1 <= top <= E or n_groups < 1 or E % n_groups or not 1 <= keep_groups <= n_groups
                or keep_groups * (E // n_groups) < top):
            raise KernelError(f"routing: {top} of {E} experts (at most {MAX_EXPERTS}) from {keep_groups} of {n_groups} groups")
        idx = torch.empty((N, top), dtype=torch.int32, device=self.device)
        weight = torch.empty((N, top), dtype=torch.float32, device=self.device)
        _check(self._hybrid().soc_moe_route(_ptr(logits), c_int(logits.stride(0) if N > 1 else E), _ptr(correction), c_int(N), c_int(E),
                                            c_int(top), c_int(n_groups), c_int(keep_groups), c_float(renorm_eps),
                                            c_int(1 if scoring == "sigmoid" else 0), c_int(group_top), c_float(scale), _ptr(idx),
                                            _ptr(weight), self._stream()),
               "moe_route")
        return idx, weight

    def moe_sort(self, idx, E, tile=EXPERT_TILE):
        """The (token, choice) pairs of ``idx`` [N, top] laid out expert by expert, in tiles of ``tile`` places: an
        ``ExpertRuns``."""
        N, top = idx.shape
        self._want(idx, "experts", torch.int32)
        if not 1 <= E <= MAX_EXPERTS:
            raise KernelError(f"{E} experts (at most {MAX_EXPERTS})")
        if tile not in (EXPERT_TILE,) + tuple(t for _, t in EXPERT_TILES_MANY):
            raise KernelError(f"tiles of {tile} places")
        M = N * top
        max_tiles = (M + tile - 1) // tile + min(E, M)
        ints = torch.empty((2 * M + E + 1 + 2 * max_tiles,), dtype=torch.int32, device=self.device)
        place, pair_at, offsets = ints[:M], ints[M:2 * M], ints[2 * M:2 * M + E + 1]
        tiles = ints[2 * M + E + 1:].view(max_tiles, 2)
        _check(self._hybrid().soc_moe_sort(_ptr(idx), c_int(M), c_int(E), c_int(tile), c_int(max_tiles), _ptr(offsets),
                                           _ptr(place), _ptr(pair_at), _ptr(tiles), self._stream()), "moe_sort")
        return ExpertRuns(place, pair_at, offsets, tiles, top, tile)

    def grouped_linear(self, x, w, runs, by_token, glu=None, out_dtype=None):
        """out[p] = w[e] x[row of p] for every place p of expert e's run; x rows are tokens (``by_token``: place p
        reads the token of its pair) or places. w [E, n_out, K]; with ``glu`` = (limit, slope[, shift = 1]) w holds
        [gate | up] rows and out [M, n_out / 2] is g sigmoid(slope g) (u + shift) with g = min(gate, limit),
        u = clamp(up, +-limit)."""
        self._want(x, "x", self.dtype)
        self._want(w, "weights per expert", self.dtype)
        M = runs.place.numel()
        E, rows, K = w.shape
        if x.shape[1] != K or (not by_token and x.shape[0] != M) or runs.offsets.numel() != E + 1:
            raise KernelError(f"products per expert: x {tuple(x.shape)}, weights {tuple(w.shape)}, {M} places")
        ff = 0
        n_out = rows
        if glu is not None:
            if rows % 2:
                raise KernelError("gate and up have the same number of rows")
            ff = n_out = rows // 2
        out_dtype = out_dtype or self.dtype
        if out_dtype not in (self.dtype, torch.float32) or (glu is not None and out_dtype != self.dtype):
            raise KernelError(f"products per expert: a result in {out_dtype}")
        out = torch.empty((M, n_out), dtype=out_dtype, device=self.device)
        limit, slope, shift = (tuple(glu) + (1.0,))[:3] if glu is not None else (0.0, 0.0, 1.0)
        _check(self._hybrid().soc_grouped_linear(
            _ptr(x), c_int(x.stride(0)), _ptr(runs.pair_at if by_token else None), c_int(runs.top), _ptr(w), _ptr(runs.offsets),
            _ptr(runs.tiles), c_int(runs.tiles.shape[0]), c_int(runs.tile), _ptr(out), c_int(n_out), c_int(K), c_int(ff), c_float(limit),
            c_float(slope), c_float(shift), c_int(1 if out_dtype == torch.float32 and self.dtype != torch.float32 else 0), c_int(self.code),
            self._stream()), "grouped_linear")
        return out

    def moe_combine(self, y, runs, weight, extra=None, extra_gate=None):
        """float32 [N, d]: each token's weighted sum of its experts' rows of ``y`` (float32 [M, d] by place), plus
        ``extra`` [N, d] (compute dtype) if given, times sigmoid(``extra_gate``) (float32 [N], which may be a column
        of a wider product) if that is given."""
        N, top = weight.shape
        d = y.shape[1]
        self._want(y, "expert results", torch.float32, (N * top, d))
        self._want(weight, "weights", torch.float32)
        if extra is not None:
            self._want(extra, "extra", self.dtype, (N, d))
        ldg = 0
        if extra_gate is not None:
            if (extra is None or extra_gate.device.type != "cuda" or extra_gate.dtype != torch.float32
                    or tuple(extra_gate.shape) != (N,)):
                raise KernelError("the gate of the extra term: float32 [N] beside an extra term")
            ldg = extra_gate.stride(0) if N > 1 else 1
        out = torch.empty((N, d), dtype=torch.float32, device=self.device)
        step = 65535
        for lo in range(0, N, step):
            n = min(step, N - lo)
            _check(self._hybrid().soc_moe_combine(_ptr(y), _ptr(runs.place[lo * top:]), _ptr(weight[lo:]),
                                                  _ptr(extra[lo:]) if extra is not None else None,
                                                  _ptr(extra_gate[lo:]) if extra_gate is not None else None, c_int(ldg),
                                                  _ptr(out[lo:]), c_int(n), c_int(d),
                                                  c_int(top), c_int(self.code), self._stream()), "moe_combine")
        return out

    def moe_experts(self, x, idx, weight, w_gate_up, w_down, limit, slope, extra=None, shift=1.0, extra_gate=None):
        """The weighted sum of each token's chosen experts (gated feed-forwards with the activation
        g sigmoid(slope g) (u + shift) under a clamp: ``w_gate_up`` [E, 2 ff, d], ``w_down`` [E, d, ff]) plus ``extra``
        (times sigmoid(``extra_gate``) per token if given); float32 [N, d]."""
        E, _, d = w_gate_up.shape
        ff = w_down.shape[2]
        # many tokens per expert, in bfloat16 with rows that start on 16 bytes: the larger tiles of the matrix cores
        # (a weight row then comes from memory once per 128 or 256 tokens of its expert)
        tile = EXPERT_TILE
        if self.dtype == torch.bfloat16 and d % 8 == 0 and ff % 8 == 0 and x.stride(0) % 8 == 0:
            tile = next((t for least, t in EXPERT_TILES_MANY if idx.numel() >= least * E), EXPERT_TILE)
        runs = self.moe_sort(idx, E, tile)
        act = self.grouped_linear(x, w_gate_up, runs, by_token=True, glu=(limit, slope, shift))
        y = self.grouped_linear(act, w_down, runs, by_token=False, out_dtype=torch.float32)
        return self.moe_combine(y, runs, weight, extra, extra_gate)

    # -- a per-token side input, and the residual sum with a cast -----------------------------------------------------
    def side_gate(self, t, table, col0, token_ids):
        """gelu_tanh(t) * table[token, col0 : col0 + dim]; t [N, dim]."""
        N, dim = t.shape
        self._want(t, "t", self.dtype)
        self._want(table, "side table", self.dtype)
        self._want(token_ids, "token ids", torch.int32, (N,))
        if table.dim() != 2 or col0 < 0 or col0 + dim > table.shape[1]:
            raise KernelError(f"side table {tuple(table.shape)} has no columns {col0} .. {col0 + dim}")
        out = torch.empty((N, dim), dtype=self.dtype, device=self.device)
        _check(self._hybrid().soc_side_gate(_ptr(t), _ptr(table), c_int(table.shape[1]), c_int(col0), _ptr(token_ids),
                                            c_int(table.shape[0]), _ptr(out), c_int(N), c_int(dim), c_int(self.code),
                                            self._stream()), "side_gate")
        return out

    def add_cast(self, residual, delta):
        """residual (float32 [N, d], in place) += delta (None, [N, d] in the compute dtype, or float32 partial sums
        [S, N, d] added in order); returns the sum in the compute dtype."""
        N, d = residual.shape
        self._want(residual, "residual", torch.float32)
        whole = parts = None
        n_parts = 0
        if delta is not None and delta.dim() == 3:
            parts, n_parts = self._want(delta, "partial sums", torch.float32, (delta.shape[0], N, d)), delta.shape[0]
        elif delta is not None:
            whole = self._want(delta, "delta", self.dtype, (N, d))
        out = torch.empty((N, d), dtype=self.dtype, device=self.device)
        _check(self._hybrid().soc_add_cast(_ptr(residual), _ptr(whole), _ptr(parts), c_int(n_parts), c_longlong(N * d), _ptr(out),
                                           c_int(self.code), self._stream()), "add_cast")
        return out
