"""Wrappers of the kernels in ``csrc/composite.hip``: norms on a branch's result with the sum and a
cast, the weighted sum over depth, what prepares window attention (biases, norms per head or over the
whole projection, rotations over interleaved pairs, turned values, page writes), the means of blocks of
keys and values, a result turned back, linear attention with a decay per head or per key channel and
token, a scaled sum of two results, and the gelu-gated activation. The library is compiled and loaded
when a model first asks for one of them."""

from __future__ import annotations

from ctypes import c_float, c_int, c_longlong

import torch

from .build import load_library
from .common import _COMPOSITE_SIGNATURES, KernelError, _check, _declare, _ptr

_NORMS = {None: 0, "head": 1, "whole": 2, "turned": 3}


class Composite:
    linear_prepare_ahead = 16       # tokens of a step's longest portion from which linear attention prepares ahead

    def _composite(self):
        lib = getattr(self, "_composite_lib", None)
        if lib is None:
            lib = self._composite_lib = load_library("composite")
            _declare(lib, _COMPOSITE_SIGNATURES)
        return lib

    # -- norms on results, and the weighted sum over depth ---------------------------------------------------
    def depth_begin(self, residual, total, cast=False):
        """float32 [total, N, d] whose first entry is ``residual``: the results by depth of one step. With ``cast``
        returns (that, the stream in the compute dtype)."""
        self._want(residual, "residual", torch.float32)
        kept = torch.empty((total,) + tuple(residual.shape), dtype=torch.float32, device=self.device)
        out = torch.empty(residual.shape, dtype=self.dtype, device=self.device) if cast else None
        _check(self._composite().soc_depth_begin(_ptr(residual), _ptr(kept), _ptr(out), c_longlong(residual.numel()),
                                                 c_int(self.code), self._stream()), "depth_begin")
        return (kept, out) if cast else kept

    def norm_add_cast(self, residual, y, gain, eps, cast=True, depth=None):
        """residual (float32 [N, d], in place) += y / rms(y) * gain, y in the compute dtype or float32; with
        ``cast`` returns the sum in the compute dtype. ``depth`` = (kept, count, weights): that sum is a layer's
        result; it is filed as kept[count] and what goes on, in residual and in what is returned, is the sum over
        j <= count of weights[j] kept[j] (``depth_average`` in the same kernel)."""
        N, d = residual.shape
        self._want(residual, "residual", torch.float32)
        if y.dtype not in (self.dtype, torch.float32):
            raise KernelError(f"a branch's result in {y.dtype}")
        self._want(y, "branch result", y.dtype, (N, d))
        self._want(gain, "norm gain", torch.float32, (d,))
        kept, count, weights = depth if depth is not None else (None, 0, None)
        if depth is not None:
            self._check_depth(kept, count, weights, N, d)
        out = torch.empty((N, d), dtype=self.dtype, device=self.device) if cast else None
        _check(self._composite().soc_norm_add_cast(_ptr(residual), _ptr(y), c_int(1 if y.dtype == torch.float32 else 0), _ptr(gain),
                                                   c_float(eps), _ptr(out), c_int(N), c_int(d), _ptr(kept), c_int(count), _ptr(weights),
                                                   c_int(self.code), self._stream()),
               "norm_add_cast")
        return out

    def _check_depth(self, kept, count, weights, N, d):
        self._want(kept, "results by depth", torch.float32)
        if kept.dim() != 3 or tuple(kept.shape[1:]) != (N, d) or not 0 < count < kept.shape[0]:
            raise KernelError(f"results by depth {tuple(kept.shape)} have no place {count} for rows of {(N, d)}")
        self._want(weights, "depth weights", torch.float32, (count + 1,))

    def depth_average(self, residual, kept, count, weights, cast=True):
        """kept[count] <- residual; residual <- sum over j <= count of weights[j] kept[j]; with ``cast`` returns
        the sum in the compute dtype."""
        N, d = residual.shape
        self._want(residual, "residual", torch.float32)
        self._check_depth(kept, count, weights, N, d)
        out = torch.empty((N, d), dtype=self.dtype, device=self.device) if cast else None
        _check(self._composite().soc_depth_average(_ptr(residual), _ptr(kept), c_int(count), _ptr(weights), _ptr(out),
                                                   c_longlong(N * d), c_int(self.code), self._stream()), "depth_average")
        return out

    # -- window attention ------------------------------------------------------------------------------------------
    def window_prepare(self, x, cols, Hq, Hkv, D, Dv, P, bias, q_gain, k_gain, norm, eps, inv_freq, rotary_dim, value_freq,
                       positions, token_rows, slot, magnitude=1.0):
        """x [N, ld] holds, from columns ``cols`` = (q, k, v) on, Hq heads of D, Hkv heads of D and Hkv heads of Dv;
        ``bias`` (float32 [ld] or None) is added to them. ``norm`` "head": q and k RMS-normed per head (gains [D]);
        "whole": over the whole of q and of k (gains [Hq D], [Hkv D]); "turned": per head behind the rotation, without
        gains; None: as they are. Pairs (2i, 2i + 1) of the first ``rotary_dim`` elements of every q and k head are
        turned by position * inv_freq[i], cosines and sines times ``magnitude``; ``slot`` None with Hkv 0: queries
        only, nothing is written; with ``value_freq``
        [Dv / 2] the pairs of every v head by position * value_freq[m]. Keys and values go to the token's place in the
        pools [pages, Hkv, block, P], zeros behind D and Dv. Returns q [N, Hq, P], zeros behind D."""
        N, ld = x.shape
        self._want(x, "x", self.dtype)
        col_q, col_k, col_v = cols
        if min(cols) < 0 or col_q + Hq * D > ld or col_k + Hkv * D > ld or col_v + Hkv * Dv > ld:
            raise KernelError(f"queries, keys and values from columns {cols} do not fit rows of {ld}")
        if not (1 <= D <= P and 1 <= Dv <= P and P <= 256) or rotary_dim % 2 or not 0 <= rotary_dim <= D:
            raise KernelError(f"head sizes {D} and {Dv} in pools of {P}, rotation over {rotary_dim}")
        if norm not in _NORMS:
            raise KernelError(f"norm {norm!r}: head, whole or None")
        if bias is not None:
            self._want(bias, "bias", torch.float32, (ld,))
        if norm in ("head", "whole"):
            self._want(q_gain, "q gain", torch.float32, (D,) if norm == "head" else (Hq * D,))
            self._want(k_gain, "k gain", torch.float32, (D,) if norm == "head" else (Hkv * D,))
        half = rotary_dim // 2
        if half:
            self._want(inv_freq, "inv_freq", torch.float32, (half,))
        if value_freq is not None:
            if Dv % 2:
                raise KernelError("turned values have an even size")
            self._want(value_freq, "value frequencies", torch.float32, (Dv // 2,))
        self._want(positions, "positions", torch.int32, (N,))
        self._want(token_rows, "token_rows", torch.int32, (N,))
        if (slot is None) != (Hkv == 0):
            raise KernelError("queries alone come with no kv heads and no cache slot")
        gains = norm in ("head", "whole")
        if slot is None:
            kp, vp, table, width, bs = None, None, None, 0, 1
        else:
            self._check_slot(slot, Hkv, P)
            kp, vp, table, width, bs = slot.k, slot.v, slot.block_table, slot.block_table.shape[1], slot.block_size
        q = torch.empty((N, Hq, P), dtype=self.dtype, device=self.device)
        _check(self._composite().soc_window_prepare(
            _ptr(x), c_int(ld), c_int(col_q), c_int(col_k), c_int(col_v), _ptr(bias), _ptr(q), _ptr(kp), _ptr(vp),
            _ptr(table), c_int(width), _ptr(token_rows), _ptr(positions),
            _ptr(q_gain if gains else None), _ptr(k_gain if gains else None), c_int(_NORMS[norm]), c_float(eps),
            _ptr(inv_freq if half else None), c_int(half), c_float(magnitude), _ptr(value_freq), c_int(N), c_int(Hq), c_int(Hkv),
            c_int(D), c_int(Dv), c_int(P), c_int(bs), c_int(self.code), self._stream()), "window_prepare")
        return q

    def pool_blocks(self, slot, ctx):
        """The mean key and value of every block of ``slot.pool`` positions whose last position is among the step's
        tokens, from the slot's pages into its pages of means (``slot.pooled``)."""
        means, per = slot.pooled, slot.pool
        if means is None or per < 1:
            raise KernelError("this cache slot keeps no means of blocks")
        Hkv, P = slot.k.shape[1], slot.k.shape[3]
        self._check_slot(slot, Hkv, P)
        self._check_slot(means, Hkv, P)
        if means.block_size != slot.block_size:
            raise KernelError("the pages of means hold as many entries as the tokens' pages")
        self._want(ctx.seq_qstart, "sequence starts", torch.int32, (ctx.n_seqs + 1,))
        self._want(ctx.seq_rows, "sequence rows", torch.int32, (ctx.n_seqs,))
        self._want(ctx.seq_ctx, "sequence lengths", torch.int32, (ctx.n_seqs,))
        _check(self._composite().soc_pool_blocks(
            _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table), c_int(slot.block_table.shape[1]), _ptr(means.k), _ptr(means.v),
            _ptr(means.block_table), c_int(means.block_table.shape[1]), _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(ctx.seq_ctx),
            c_int(ctx.n_seqs), c_int(max(1, ctx.max_q_len)), c_int(Hkv), c_int(P), c_int(slot.block_size), c_int(per),
            c_int(self.code), self._stream()), "pool_blocks")

    def turn_back(self, o, H, P, Dv, value_freq, positions):
        """o [N, H * P] -> [N, H * Dv]: the first Dv elements of each head, pairs (2m, 2m + 1) turned by
        -position * value_freq[m] (None: as they are)."""
        N = o.shape[0]
        self._want(o, "o", self.dtype, (N, H * P))
        if Dv > P:
            raise KernelError(f"{Dv} elements of heads of {P}")
        if value_freq is not None:
            self._want(value_freq, "value frequencies", torch.float32, (Dv // 2,))
            self._want(positions, "positions", torch.int32, (N,))
        out = torch.empty((N, H * Dv), dtype=self.dtype, device=self.device)
        _check(self._composite().soc_turn_back(_ptr(o), _ptr(out), _ptr(positions), _ptr(value_freq), c_int(N), c_int(H), c_int(P),
                                               c_int(Dv), c_int(self.code), self._stream()), "turn_back")
        return out

    # -- linear attention ----------------------------------------------------------------------------------------
    def linear_attention(self, x, cols, H, D, Dv, q_scale, activate, decays, z, z_bias, tau, state, offset, ctx,
                         prepared=None, ones=0):
        """S <- diag(decay) S + k v^T, o = S^T q per head over each sequence's tokens, from and into the row's state
        ([H, D, Dv] from ``offset``). x [N, ld] holds q and k (H heads of D) and v (H heads of Dv) from columns
        ``cols`` on; with ``activate`` they pass silu; q is scaled by ``q_scale``. The decay is ``decays`` [H], or, with
        ``z`` (float32 [N, H D]), sigmoid(z + z_bias)^(1 / tau) per token and key channel. float32 [N, H * Dv].
        ``prepared`` (float32 [N, 3, H D]): q, k and the decays per token, head and key channel as the caller made them
        (x then gives the values only). ``ones``: the last that many of the Dv value columns are not in x, whose heads
        hold Dv - ones, and read 1 (a sum of the keys beside the state)."""
        N, ld = x.shape
        self._want(x, "x", self.dtype)
        col_q, col_k, col_v = cols
        if not 0 <= ones < Dv:
            raise KernelError(f"{ones} columns of ones among {Dv}")
        if min(cols) < 0 or max(col_q, col_k) + H * D > ld or col_v + H * (Dv - ones) > ld:
            raise KernelError(f"queries, keys and values from columns {cols} do not fit rows of {ld}")
        if not 1 <= D <= 256 or Dv < 1:
            raise KernelError(f"linear attention: heads of {D} and {Dv}")
        if prepared is not None:
            if z is not None or decays is not None or activate:
                raise KernelError("linear attention: prepared q, k and decays come alone")
            self._want(prepared, "prepared q, k and decays", torch.float32, (N, 3, H * D))
        elif (z is None) == (decays is None):
            raise KernelError("linear attention: a decay per head, or per token and key channel")
        if z is not None:
            self._want(z, "decay logits", torch.float32, (N, H * D))
            self._want(z_bias, "decay bias", torch.float32, (H * D,))
            if not tau > 0:
                raise KernelError("tau is positive")
        elif prepared is None:
            self._want(decays, "decays", torch.float32, (H,))
        stride = self._state(state, offset, H * D * Dv, ctx)
        out = torch.empty((N, H * Dv), dtype=torch.float32, device=self.device)
        # a step with a portion of some length: activations, the scale and the decays are taken once, ahead of the
        # walk (each of a head's workgroups would take them again); single tokens and short portions where they
        # are staged
        prep = prepared
        if prepared is None and (activate or z is not None) and ctx.max_q_len >= self.linear_prepare_ahead:
            prep = torch.empty((N, 3 if z is not None else 2, H * D), dtype=torch.float32, device=self.device)
        _check(self._composite().soc_linear_attention(
            _ptr(x), c_int(ld), c_int(col_q), c_int(col_k), c_int(col_v), c_float(q_scale), c_int(1 if activate else 0),
            _ptr(decays), _ptr(z), _ptr(z_bias), c_float(tau), c_int(H), c_int(D), c_int(Dv), _ptr(state), stride, c_int(offset),
            _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(prep), c_int(1 if prepared is not None else 0), c_int(ones), c_int(N),
            _ptr(out), c_int(ctx.n_seqs), c_int(ctx.max_q_len), c_int(self.code), self._stream()), "linear_attention")
        return out

    # -- sums and activations ----------------------------------------------------------------------------------------
    def scaled_sum(self, a, a_scale, b, b_scale, bias=None):
        """float32 [N, d]: a_scale * (a + bias) + b_scale * b; a and b in the compute dtype or float32, ``b`` and
        ``bias`` (float32 [d]) may be None."""
        N, d = a.shape
        for name, t in (("a", a), ("b", b)):
            if t is not None:
                if t.dtype not in (self.dtype, torch.float32):
                    raise KernelError(f"scaled sum: {name} in {t.dtype}")
                self._want(t, name, t.dtype, (N, d))
        if bias is not None:
            self._want(bias, "bias", torch.float32, (d,))
        out = torch.empty((N, d), dtype=torch.float32, device=self.device)
        _check(self._composite().soc_scaled_sum(
            _ptr(a), c_int(1 if a.dtype == torch.float32 else 0), c_float(a_scale), _ptr(b),
            c_int(1 if b is not None and b.dtype == torch.float32 else 0), c_float(b_scale), _ptr(bias), _ptr(out), c_int(N), c_int(d),
            c_int(self.code), self._stream()), "scaled_sum")
        return out

    def glu_gelu(self, gate_up, ff):
        """[N, gate | up] -> gelu_tanh(gate) * up; gate and up are the first 2 ff columns."""
        self._want(gate_up, "gate and up", self.dtype)
        N, ld = gate_up.shape
        if ff < 1 or 2 * ff > ld:
            raise KernelError(f"{ld} columns do not hold gate and up of {ff}")
        out = torch.empty((N, ff), dtype=self.dtype, device=self.device)
        _check(self._composite().soc_glu_gelu(_ptr(gate_up), _ptr(out), c_int(N), c_int(ff), c_int(ld), c_int(self.code),
                                              self._stream()), "glu_gelu")
        return out
