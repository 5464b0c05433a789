"""Wrappers of the kernels in ``csrc/memory.hip``: the gates of a matrix memory with their running maximum and
what they make of q, k and the decays ahead of the recurrence; the denominators, head norms, gain and gate behind
it; and the two maps of differential attention combined. The library is compiled and loaded when a model first asks
for one of them."""

from __future__ import annotations

from ctypes import c_float, c_int

import torch

from .build import load_library
from .common import _MEMORY_SIGNATURES, KernelError, _check, _declare, _ptr


class Memory:
    def _memory(self):
        lib = getattr(self, "_memory_lib", None)
        if lib is None:
            lib = self._memory_lib = load_library("memory")
            _declare(lib, _MEMORY_SIGNATURES)
        return lib

    def memory_gates(self, gates, bias, cap, x, cols, H, D, q_scale, state, offset, ctx):
        """gates float32 [N, 2 H]: logits of the input gates and, behind them, of the forget gates; ``bias`` [2 H].
        i = cap tanh((z_i + b_i) / cap), f = logsigmoid(cap tanh((z_f + b_f) / cap)); per sequence and head, from the
        maximum that the row's state holds at ``offset`` + head: m' = max(f + m, i), keep = exp(f + m - m'),
        take = exp(i - m'). x [N, ld] holds q and k (H heads of D) from columns ``cols`` = (q, k, .) on. Returns
        (float32 [N, 3, H D]: q * q_scale, k * take, keep for every key channel; the maxima m', float32 [N, H]) and
        leaves each row's last maximum in its state."""
        N, ld = x.shape
        self._want(x, "x", self.dtype)
        self._want(gates, "gate logits", torch.float32, (N, 2 * H))
        self._want(bias, "gate bias", torch.float32, (2 * H,))
        col_q, col_k = cols[0], cols[1]
        if min(col_q, col_k) < 0 or max(col_q, col_k) + H * D > ld or D < 1 or not cap > 0:
            raise KernelError(f"matrix memory: q and k from columns {(col_q, col_k)} of rows of {ld}, {H} heads of {D}, cap {cap}")
        stride = self._state(state, offset, H, ctx)
        scratch = torch.empty((3, N, H), dtype=torch.float32, device=self.device)
        prep = torch.empty((N, 3, H * D), dtype=torch.float32, device=self.device)
        _check(self._memory().soc_memory_gates(
            _ptr(gates), _ptr(bias), c_float(cap), _ptr(x), c_int(ld), c_int(col_q), c_int(col_k), c_float(q_scale), c_int(H),
            c_int(D), _ptr(state), stride, c_int(offset), _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), c_int(ctx.n_seqs), c_int(max(1, ctx.max_q_len)), c_int(N),
            _ptr(scratch[0]), _ptr(scratch[1]), _ptr(scratch[2]), _ptr(prep), c_int(self.code), self._stream()), "memory_gates")
        return prep, scratch[0]

    def memory_finish(self, raw, maxima, z, gain, H, Dv, eps, den_eps):
        """raw float32 [N, H (Dv + 1)]: per head S^T q and, last, n . q. Each head's first Dv elements over
        max(|n . q|, exp(-maximum)) + den_eps, then over their root mean square, times ``gain`` [H Dv], times
        sigmoid(z[:, :H Dv]) (``z`` in the compute dtype, it may be wider); [N, H Dv] in the compute dtype."""
        N = raw.shape[0]
        self._want(raw, "the recurrence's result", torch.float32, (N, H * (Dv + 1)))
        self._want(maxima, "maxima", torch.float32, (N, H))
        self._want(z, "gate logits", self.dtype)
        self._want(gain, "gain", torch.float32, (H * Dv,))
        if z.dim() != 2 or z.shape[0] != N or z.shape[1] < H * Dv:
            raise KernelError(f"gate logits {tuple(z.shape)} against {N} rows of {H * Dv}")
        out = torch.empty((N, H * Dv), dtype=self.dtype, device=self.device)
        _check(self._memory().soc_memory_finish(_ptr(raw), _ptr(maxima), _ptr(z), c_int(z.shape[1]), _ptr(gain), c_int(N), c_int(H),
                                                c_int(Dv), c_float(eps), c_float(den_eps), _ptr(out), c_int(self.code),
                                                self._stream()), "memory_finish")
        return out

    def diff_combine(self, o, H, G, P, Dv, lam, eps, out_scale):
        """o [N, 2 H * P]: attention results laid out (kv head, map, query head of the group), heads of P. Head h's
        first Dv elements become (a1 - lam a2) over their root mean square times out_scale; [N, H Dv]."""
        N = o.shape[0]
        self._want(o, "o", self.dtype, (N, 2 * H * P))
        if G < 1 or H % G or not 1 <= Dv <= P:
            raise KernelError(f"differential attention: {H} heads in {G} groups, {Dv} of {P} elements")
        out = torch.empty((N, H * Dv), dtype=self.dtype, device=self.device)
        _check(self._memory().soc_diff_combine(_ptr(o), _ptr(out), c_int(N), c_int(H), c_int(G), c_int(P), c_int(Dv), c_float(lam),
                                               c_float(eps), c_float(out_scale), c_int(self.code), self._stream()), "diff_combine")
        return out
