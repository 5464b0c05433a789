"""Wrappers of the kernels in ``csrc/mixers.hip``: blocks with norms on both sides of a branch,
mixers that carry a state per row, and attention over a cached latent. The library is compiled
and loaded when a model first asks for one of them."""

from __future__ import annotations

from ctypes import c_float, c_int, c_longlong

import torch

from .build import load_library
from .common import _DTYPE_CODE, _MIXER_SIGNATURES, KernelError, _check, _declare, _ptr


class Mixers:
    def _mixers(self):
        lib = getattr(self, "_mixers_lib", None)
        if lib is None:
            lib = self._mixers_lib = load_library("mixers")
            _declare(lib, _MIXER_SIGNATURES)
        return lib

    # -- blocks ----------------------------------------------------------------------------------
    def gated_norm_add(self, residual, y, gate_logits, gate_bias, gain, eps, mult, next_gain=None, next_eps=0.0, y_bias=None):
        """residual (float32 [N, d], in place) += mult * gain * g / rms(g) with g = y *
        sigmoid(gate_logits + gate_bias) (no gate: g = y). With ``next_gain``: returns
        residual / rms(residual) * next_gain in the compute dtype; else None. ``gate_logits`` may be
        [N, d] columns of a wider product (rows apart by its width). ``y`` is in the compute dtype or float32;
        ``y_bias`` (float32 [d]) is added to it first."""
        N, d = residual.shape
        self._want(residual, "residual", torch.float32)
        if y.dtype not in (self.dtype, torch.float32):
            raise KernelError(f"a branch's result in {y.dtype}")
        self._want(y, "branch result", y.dtype, (N, d))
        if y_bias is not None:
            self._want(y_bias, "the result's bias", torch.float32, (d,))
        self._want(gain, "norm gain", torch.float32, (d,))
        ldg = 0
        if gate_logits is not None:
            if (gate_logits.device.type != "cuda" or gate_logits.dtype != self.dtype or tuple(gate_logits.shape) != (N, d)
                    or gate_logits.stride(1) != 1 or gate_logits.stride(0) < d):
                raise KernelError(f"gate logits {tuple(gate_logits.shape)} with strides {gate_logits.stride()} do not fit [{N}, {d}]")
            ldg = gate_logits.stride(0)
            self._want(gate_bias, "gate bias", torch.float32, (d,))
        out = None
        if next_gain is not None:
            self._want(next_gain, "next norm's gain", torch.float32, (d,))
            out = torch.empty((N, d), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_gated_norm_add(
            _ptr(residual), _ptr(y), c_int(1 if y.dtype == torch.float32 else 0), _ptr(y_bias), _ptr(gate_logits), c_int(ldg), _ptr(gate_bias if gate_logits is not None else None), _ptr(gain),
            c_float(eps), c_float(mult), _ptr(next_gain), c_float(next_eps), _ptr(out), c_int(N), c_int(d),
            c_int(self.code), self._stream()), "gated_norm_add")
        return out

    def glu_clamped(self, gate_up, limit, slope, ff=None):
        """[N, gate | up] -> g * sigmoid(slope g) * (u + 1), g = min(gate, limit), u = clamp(up, +-limit).
        With ``ff``: gate and up are the first 2 ff columns of a wider product."""
        self._want(gate_up, "gate and up", self.dtype)
        N, ld = gate_up.shape
        if ff is None:
            if ld % 2:
                raise KernelError("gate and up have the same number of columns")
            ff = ld // 2
        if ff < 1 or 2 * ff > ld:
            raise KernelError(f"{ld} columns do not hold gate and up of {ff}")
        out = torch.empty((N, ff), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_glu_clamped(_ptr(gate_up), _ptr(out), c_int(N), c_int(ff), c_int(ld), c_float(limit),
                                              c_float(slope), c_int(self.code), self._stream()), "glu_clamped")
        return out

    # -- state per row ---------------------------------------------------------------------------------
    def _state(self, state, offset, length, ctx):
        self._want(state, "state", torch.float32)
        if state.dim() != 2 or offset < 0 or offset + length > state.shape[1]:
            raise KernelError(f"a row's state of {tuple(state.shape)} does not hold {length} elements from {offset}")
        self._want(ctx.seq_qstart, "sequence starts", torch.int32, (ctx.n_seqs + 1,))
        self._want(ctx.seq_rows, "sequence rows", torch.int32, (ctx.n_seqs,))
        return c_longlong(state.shape[1])

    def token_shift(self, h, mu, state, offset, ctx):
        """[S, N, d]: h + (previous token's h - h) * mu[s]; the row's state (d elements from
        ``offset``) holds the input of the last token before the step, and after it the step's last."""
        N, d = h.shape
        self._want(h, "h", self.dtype)
        S = mu.shape[0]
        self._want(mu, "blend weights", torch.float32, (S, d))
        stride = self._state(state, offset, d, ctx)
        out = torch.empty((S, N, d), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_token_shift(_ptr(h), _ptr(mu), c_int(S), _ptr(state), stride, c_int(offset),
                                              _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(out), c_int(N), c_int(d),
                                              c_int(ctx.n_seqs), c_int(ctx.max_q_len), c_int(self.code), self._stream()),
               "token_shift")
        return out

    def wkv_decay(self, t, w2_t, w0):
        """float32 [N, C]: exp(-exp(tanh(t) w2 + w0)); t float32 [N, rank], ``w2_t`` [rank, C] (the stored
        matrix transposed, so that consecutive outputs read consecutive elements)."""
        N, rank = t.shape
        self._want(t, "decay latent", torch.float32)
        w2 = self._want(w2_t, "decay matrix")
        C = w2.shape[1]
        if w2.shape != (rank, C) or w2.dtype not in _DTYPE_CODE or rank > 8192:
            raise KernelError(f"decay matrix {tuple(w2.shape)} does not fit a latent of {rank}")
        self._want(w0, "decay bias", torch.float32, (C,))
        out = torch.empty((N, C), dtype=torch.float32, device=self.device)
        _check(self._mixers().soc_wkv_decay(_ptr(t), _ptr(w2), _ptr(w0), _ptr(out), c_int(N), c_int(C), c_int(rank),
                                            c_int(_DTYPE_CODE[w2.dtype]), self._stream()), "wkv_decay")
        return out

    def wkv(self, r, k, v, decay, g, bonus, gain, eps, H, state, offset, ctx):
        """The recurrence with a decay per key channel over each sequence's tokens, from and into
        the row's state ([H, D, D] from ``offset``); each head's result over its root mean square,
        times ``gain``, times silu(g). [N, H * D] in the compute dtype."""
        N, C = r.shape
        if C % H or not 1 <= C // H <= 256:
            raise KernelError(f"{C} channels in {H} heads: head sizes run from 1 to 256")
        D = C // H
        for t, name in ((r, "r"), (k, "k"), (v, "v"), (g, "g")):
            self._want(t, name, self.dtype, (N, C))
        self._want(decay, "decay", torch.float32, (N, C))
        self._want(bonus, "bonus", torch.float32, (H, D))
        self._want(gain, "gain", torch.float32, (C,))
        stride = self._state(state, offset, H * D * D, ctx)
        raw = torch.empty((N, C), dtype=torch.float32, device=self.device)
        _check(self._mixers().soc_wkv(_ptr(r), _ptr(k), _ptr(v), _ptr(decay), _ptr(bonus), c_int(H), c_int(D), _ptr(state),
                                      stride, c_int(offset), _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(raw),
                                      c_int(ctx.n_seqs), c_int(ctx.max_q_len), c_int(self.code), self._stream()), "wkv")
        # (a head's columns are spread over workgroups: its norm is a kernel of its own)
        return self.gated_group_norm(raw, g, gain, H, eps, gate_first=False)

    def causal_conv_silu(self, x, col, C, weight, bias, state, offset, ctx):
        """silu of a causal convolution per channel over columns col .. col + C of ``x``; the row's
        state ([taps - 1, C] from ``offset``) holds the inputs before the step. [N, C]."""
        self._want(x, "x", self.dtype)
        N, ldx = x.shape
        taps = weight.shape[1]
        self._want(weight, "taps", torch.float32, (C, taps))
        self._want(bias, "bias", torch.float32, (C,))
        if col < 0 or col + C > ldx or not 1 <= taps <= 33:
            raise KernelError(f"convolution: columns {col}..{col + C} of {ldx}, {taps} taps (at most 33)")
        stride = self._state(state, offset, (taps - 1) * C, ctx)
        out = torch.empty((N, C), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_causal_conv_silu(
            _ptr(x), c_int(ldx), c_int(col), c_int(C), _ptr(weight), _ptr(bias), c_int(taps), _ptr(state), stride,
            c_int(offset), _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows), _ptr(out), c_int(ctx.n_seqs), c_int(ctx.max_q_len),
            c_int(self.code), self._stream()), "causal_conv_silu")
        return out

    def ssd(self, xbc, dt, dt_bias, a_log, skip, H, P, Ns, G, state, offset, ctx):
        """The recurrence with a scalar decay per head over each sequence's tokens; xbc [N, x | B | C],
        dt float32 [N, H] before bias and softplus; the row's state is [H, Ns, P] from ``offset``.
        float32 [N, H * P]."""
        N = xbc.shape[0]
        self._want(xbc, "x, B, C", self.dtype, (N, H * P + 2 * G * Ns))
        self._want(dt, "step sizes", torch.float32, (N, H))
        for t, name in ((dt_bias, "dt bias"), (a_log, "A_log"), (skip, "D")):
            self._want(t, name, torch.float32, (H,))
        if H % G or not 1 <= Ns <= 256 or P < 1:
            raise KernelError(f"ssd: {H} heads in {G} groups, state {Ns}, head size {P}")
        stride = self._state(state, offset, H * Ns * P, ctx)
        out = torch.empty((N, H * P), dtype=torch.float32, device=self.device)
        _check(self._mixers().soc_ssd(_ptr(xbc), _ptr(dt), _ptr(dt_bias), _ptr(a_log), _ptr(skip), c_int(H), c_int(P), c_int(Ns),
                                      c_int(G), _ptr(state), stride, c_int(offset), _ptr(ctx.seq_qstart), _ptr(ctx.seq_rows),
                                      _ptr(out), c_int(ctx.n_seqs), c_int(ctx.max_q_len), c_int(self.code), self._stream()), "ssd")
        return out

    def gated_group_norm(self, y, z, gain, groups, eps, gate_first=True, sigmoid=False):
        """y (float32 [N, inner]) * silu(z[:, :inner]), RMS-normed in ``groups`` equal parts, times gain;
        ``gate_first`` False: y normed, times gain, and only then times silu(z). ``sigmoid``: the gate is
        sigmoid(z) in place of silu(z)."""
        N, inner = y.shape
        self._want(y, "y", torch.float32)
        self._want(z, "z", self.dtype)
        self._want(gain, "gain", torch.float32, (inner,))
        if z.dim() != 2 or z.shape[0] != N or z.shape[1] < inner or groups < 1 or inner % groups:
            raise KernelError(f"gated norm: z {tuple(z.shape)} against y {tuple(y.shape)} in {groups} parts")
        out = torch.empty((N, inner), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_gated_group_norm(_ptr(y), _ptr(z), c_int(z.shape[1]), _ptr(gain), c_int(N), c_int(inner),
                                                   c_int(groups), c_float(eps), c_int(1 if gate_first else 0), c_int(1 if sigmoid else 0),
                                                   _ptr(out),
                                                   c_int(self.code), self._stream()),
               "gated_group_norm")
        return out

    # -- attention over a cached latent ---------------------------------------------------------------------
    def _columns(self, x, name, N, dim):
        """``x`` is [N, dim] in the compute dtype, rows contiguous and apart by at least ``dim`` (columns of a
        wider product)."""
        if (x.device.type != "cuda" or x.dtype != self.dtype or tuple(x.shape) != (N, dim) or x.stride(1) != 1
                or x.stride(0) < dim):
            raise KernelError(f"{name}: {tuple(x.shape)} with strides {x.stride()} does not fit [{N}, {dim}]")

    def rmsnorm_cols(self, x, weight, eps):
        """RMS norm of ``x`` [N, dim], which may be columns of a wider product; returns contiguous rows."""
        N, dim = x.shape
        self._columns(x, "x", N, dim)
        self._want(weight, "norm weight", torch.float32, (dim,))
        out = torch.empty((N, dim), dtype=self.dtype, device=self.device)
        _check(self._mixers().soc_rmsnorm_cols(_ptr(x), c_int(x.stride(0)), _ptr(weight), _ptr(out), c_int(N), c_int(dim),
                                               c_float(eps), c_int(self.code), self._stream()), "rmsnorm_cols")
        return out

    def latent_write(self, kvd, R, Dr, gain, eps, inv_freq, positions, token_rows, slot):
        """kvd [N, R + Dr] (it may be columns of a wider product): the first R RMS-normed, the rest turned by
        position, into each token's place of the pool [pages, 1, block, width]."""
        N = kvd.shape[0]
        self._columns(kvd, "latent and key part", N, R + Dr)
        self._want(gain, "latent gain", torch.float32, (R,))
        self._want(inv_freq, "inv_freq", torch.float32)
        self._want(positions, "positions", torch.int32, (N,))
        self._want(token_rows, "token_rows", torch.int32, (N,))
        self._want(slot.k, "latent pool", self.dtype)
        self._want(slot.block_table, "block table", torch.int32)
        width = slot.k.shape[-1]
        if slot.k.dim() != 4 or slot.k.shape[1] != 1 or slot.k.shape[2] != slot.block_size or R + Dr > width \
                or 2 * inv_freq.numel() > Dr:
            raise KernelError(f"latent pool {tuple(slot.k.shape)} does not fit {R} + {Dr} elements per token")
        _check(self._mixers().soc_latent_write(
            _ptr(kvd), c_int(kvd.stride(0)), c_int(N), c_int(R), c_int(Dr), _ptr(gain), c_float(eps), _ptr(inv_freq),
            c_int(inv_freq.numel()),
            _ptr(positions), _ptr(token_rows), _ptr(slot.block_table), c_int(slot.block_table.shape[1]), _ptr(slot.k),
            c_int(slot.block_size), c_int(width), c_int(self.code), self._stream()), "latent_write")

    def head_linear(self, x, K, w, out=None, ldo=None):
        """out[n, h, :n_out] = x[n, h, :K] w[h]^T; x [N, H, ldx], w [H, n_out, K]."""
        N, H, ldx = x.shape
        self._want(x, "x", self.dtype)
        self._want(w, "weights per head", self.dtype)
        n_out = w.shape[1]
        if w.shape != (H, n_out, K) or K > ldx:
            raise KernelError(f"per-head product: weights {tuple(w.shape)} against {H} heads of {K} (of {ldx})")
        if out is None:
            out = torch.empty((N, H, n_out), dtype=self.dtype, device=self.device)
        self._want(out, "out", self.dtype)
        if out.dim() != 3 or out.shape[:2] != (N, H) or out.shape[2] < n_out:
            raise KernelError(f"per-head product: out {tuple(out.shape)}")
        if (self.dtype == torch.bfloat16 and N > 16 and self.library_gemm and K % 8 == 0 and n_out % 8 == 0
                and not self._tuning and not torch.cuda.is_current_stream_capturing()):
            # more than 16 rows in bfloat16: the library's batched product, as for every other
            # product of that size (float32 sums inside), from operands laid out by head (never while the
            # library times its solutions: its tuning pass is kept to plain products); its [H, N, n_out]
            # result is laid back by head
            by_head = x.transpose(0, 1)[:, :, :K].contiguous()
            out[:, :, :n_out].copy_(torch.bmm(by_head, w.transpose(1, 2)).transpose(0, 1))
            return out
        _check(self._mixers().soc_head_linear(_ptr(x), c_int(ldx), _ptr(w), _ptr(out), c_int(out.shape[2]), c_int(N), c_int(H),
                                              c_int(n_out), c_int(K), c_int(self.code), self._stream()), "head_linear")
        return out

    def latent_query(self, q, H, D, Dr, w_uk_t, width, inv_freq, positions):
        """q [N, H * (D + Dr)] -> [N, H, width]: per head [w_uk_t[h] q_plain | q_rot turned by position | zeros]."""
        N = q.shape[0]
        self._want(q, "q", self.dtype, (N, H * (D + Dr)))
        R = w_uk_t.shape[1]
        self._want(positions, "positions", torch.int32, (N,))
        self._want(inv_freq, "inv_freq", torch.float32)
        if R + Dr > width or 2 * inv_freq.numel() > Dr:
            raise KernelError(f"folded query of {R} + {Dr} does not fit {width}")
        out = torch.empty((N, H, width), dtype=self.dtype, device=self.device)
        self.head_linear(q.view(N, H, D + Dr), D, w_uk_t, out)
        _check(self._mixers().soc_latent_query_turn(_ptr(q), c_int(N), c_int(H), c_int(D), c_int(Dr), c_int(R), c_int(width),
                                                    _ptr(inv_freq), c_int(inv_freq.numel()), _ptr(positions), _ptr(out),
                                                    c_int(self.code), self._stream()), "latent_query")
        return out

    def head_project(self, x, w):
        """x [N, H, ldx] (its first K read), w [H, n_out, K] -> [N, H * n_out]."""
        out = self.head_linear(x, w.shape[2], w)
        return out.view(x.shape[0], -1)
