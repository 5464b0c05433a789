"""The kernel set in plain PyTorch, for tests only.

Two uses: the per-kernel reference that each HIP kernel is compared with on the
GPU, and a stand-in kernel set that lets the step function, the cache and the
scheduler run on a CPU in the ``not gpu`` tests. Nothing in ``socrates_amd``
imports this file. Statistics, softmax, angles and sums are float32 (float64 if
the set is built with it) and results are rounded once to the compute dtype, as
the HIP kernels do.
"""

import numpy as np
import torch


def splitmix64(x: int) -> int:
    """One step of the splitmix64 generator: a counter-based hash on 64 bits."""
    m = (1 << 64) - 1
    x = (x + 0x9E3779B97F4A7C15) & m
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & m
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & m
    return x ^ (x >> 31)


def uniform_of(seed: int, draw: int) -> float:
    """The uniform number in [0, 1) that request stream ``seed`` yields at draw ``draw``."""
    h = splitmix64(splitmix64(int(seed)) ^ ((int(draw) * 0xD1342543DE82EF95) & ((1 << 64) - 1)))
    return (h >> 40) * (1.0 / (1 << 24))


class TorchKernels:
    def __init__(self, dtype=torch.float32, device="cpu", acc=torch.float32):
        self.dtype, self.device, self.acc = dtype, torch.device(device), acc

    # -- elementwise and norms ---------------------------------------------------------------
    def embedding(self, ids, table):
        return table[ids.long()].to(torch.float32 if self.acc == torch.float32 else self.acc)

    def _norm(self, x, weight, eps):
        x = x.to(self.acc)
        var = x.pow(2).mean(-1, keepdim=True)
        return x / torch.sqrt(var + eps) * weight.to(self.acc)

    def add_rmsnorm(self, residual, delta, weight, eps, rows=None):
        if delta is not None and delta.dim() == 3:            # split-K partial sums
            delta = delta.sum(0)
        if rows is not None:
            r = residual[rows.long()].to(self.acc)
            if delta is not None:
                r = r + delta[rows.long()].to(self.acc)
            return self._norm(r, weight, eps).to(self.dtype)
        if delta is not None:
            residual += delta.to(residual.dtype)
        return self._norm(residual, weight, eps).to(self.dtype)

    def rmsnorm(self, x, weight, eps):
        return self._norm(x, weight, eps).to(x.dtype)

    def scale_softcap_(self, x, scale=1.0, softcap=None):
        x.mul_(scale)
        if softcap is not None:
            x.copy_(softcap * torch.tanh(x / softcap))
        return x

    def swiglu(self, gate_up, interleave=0):
        ff = gate_up.shape[-1] // 2
        if interleave:
            blocks = gate_up.reshape(*gate_up.shape[:-1], ff // interleave, 2, interleave)
            g, u = blocks[..., 0, :].reshape(*gate_up.shape[:-1], ff), blocks[..., 1, :].reshape(*gate_up.shape[:-1], ff)
        else:
            g, u = gate_up[..., :ff], gate_up[..., ff:]
        g, u = g.to(self.acc), u.to(self.acc)
        return (u * (g * torch.sigmoid(g))).to(self.dtype)

    def linear_swiglu(self, x, w_gate_up, interleave=0):
        return self.swiglu(self.linear(x, w_gate_up), interleave)

    def linear(self, x, w, out_dtype=None, allow_partial=False):
        y = x.to(self.acc) @ w.to(self.acc).T
        return y.to(out_dtype or self.dtype)

    # -- attention pieces --------------------------------------------------------------------
    def _rotate(self, x, positions, inv_freq, rotary_dim):
        """x: [N, H, D] in acc dtype."""
        ang = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
        cos, sin = ang.cos().to(self.acc)[:, None, :], ang.sin().to(self.acc)[:, None, :]
        h = rotary_dim // 2
        x1, x2 = x[..., :h], x[..., h:rotary_dim]
        out = x.clone()
        out[..., :h] = x1 * cos - x2 * sin
        out[..., h:rotary_dim] = x2 * cos + x1 * sin
        return out

    def qk_norm_split(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps):
        N = qkv.shape[0]
        q = qkv[:, :Hq * D].reshape(N, Hq, D)
        k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(N, Hkv, D)
        v = qkv[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].reshape(N, Hkv, D).contiguous()
        if q_gain is not None:
            q = self._norm(q, q_gain, eps).to(self.dtype)
            k = self._norm(k, k_gain, eps).to(self.dtype)
        return q.contiguous(), k.contiguous(), v

    def rope(self, x, positions, inv_freq, rotary_dim):
        x.copy_(self._rotate(x.to(self.acc), positions, inv_freq, rotary_dim).to(x.dtype))

    def kv_write(self, k, v, positions, token_rows, slot):
        bs = slot.block_size
        pos = positions.long()
        page = slot.block_table[token_rows.long(), pos // bs].long()
        slot.k[page, :, pos % bs] = k.to(slot.k.dtype)
        slot.v[page, :, pos % bs] = v.to(slot.v.dtype)

    def qk_norm_rope_write(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps, inv_freq, rotary_dim,
                           positions, token_rows, slot):
        N = qkv.shape[0]
        q = qkv[:, :Hq * D].reshape(N, Hq, D).to(self.acc)
        k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(N, Hkv, D).to(self.acc)
        v = qkv[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].reshape(N, Hkv, D)
        if q_gain is not None:
            q, k = self._norm(q, q_gain, eps), self._norm(k, k_gain, eps)
        if inv_freq is not None:
            q = self._rotate(q, positions, inv_freq, rotary_dim)
            k = self._rotate(k, positions, inv_freq, rotary_dim)
        if slot is not None:
            self.kv_write(k, v, positions, token_rows, slot)
        return q.to(self.dtype).contiguous()

    def paged_attention(self, q, slot, ctx, scale, window, terms=None):
        """Token by token: gather the row's keys 0..p through the table, mask the window.
        ``terms``: a bias by distance (``slopes`` [Hq]), a soft cap of the scores, one more
        logit per head in the softmax's sum (``sinks`` [Hq]), first keys that stay visible
        behind a window (``keep_first``)."""
        terms = terms or {}
        N, Hq, D = q.shape
        Hkv, bs = slot.k.shape[1], slot.block_size
        G = Hq // Hkv
        out = torch.empty((N, Hq * D), dtype=self.dtype, device=q.device)
        table = slot.block_table.cpu().numpy()
        positions = ctx.positions.cpu().numpy()
        rows = ctx.token_rows.cpu().numpy()
        for t in range(N):
            p, row = int(positions[t]), int(rows[t])
            lo = 0 if window is None else max(0, p - window + 1)
            idx = np.arange(lo, p + 1)
            if window is not None and terms.get("keep_first"):
                idx = np.concatenate([np.arange(0, min(int(terms["keep_first"]), lo)), idx])
            pages = torch.as_tensor(table[row, idx // bs].astype(np.int64), device=q.device)
            offs = torch.as_tensor(idx % bs, device=q.device)
            k = slot.k[pages, :, offs].to(self.acc)          # [n, Hkv, D]
            v = slot.v[pages, :, offs].to(self.acc)
            if terms.get("pooled") is not None and window is not None:
                # the means of the blocks that end before the window begins, in front of the window's keys
                means, per = terms["pooled"].pooled, terms["pooled"].pool
                blocks = np.arange(max(0, (p - window + 1) // per))
                mtable = means.block_table.cpu().numpy()
                mp = torch.as_tensor(mtable[row, blocks // bs].astype(np.int64), device=q.device)
                mo = torch.as_tensor(blocks % bs, device=q.device)
                k = torch.cat([means.k[mp, :, mo].to(self.acc), k], dim=0)
                v = torch.cat([means.v[mp, :, mo].to(self.acc), v], dim=0)
                idx = np.concatenate([blocks, idx])
            qt = q[t].to(self.acc).view(Hkv, G, D)
            s = torch.einsum("hgd,nhd->hgn", qt, k) * scale
            if terms.get("slopes") is not None:
                dist = torch.as_tensor(idx - p, device=q.device).to(self.acc)
                s = s + terms["slopes"].to(self.acc).view(Hkv, G, 1) * dist
            if terms.get("softcap"):
                s = terms["softcap"] * torch.tanh(s / terms["softcap"])
            if terms.get("sinks") is not None:
                s = torch.cat([s, terms["sinks"].to(self.acc).view(Hkv, G, 1)], dim=-1)
                a = torch.softmax(s, dim=-1)[..., :-1]
            else:
                a = torch.softmax(s, dim=-1)
            out[t] = torch.einsum("hgn,nhd->hgd", a, v).reshape(Hq * D).to(self.dtype)
        return out

    # -- what closes a branch of a block with norms on both sides ------------------------------
    def gated_norm_add(self, residual, y, gate_logits, gate_bias, gain, eps, mult, next_gain=None, next_eps=0.0, y_bias=None):
        y = y.to(self.acc)
        if y_bias is not None:
            y = y + y_bias.to(self.acc)
        if gate_logits is not None:
            y = y * torch.sigmoid(gate_logits.to(self.acc) + gate_bias.to(self.acc))
        residual += (mult * self._norm(y, gain, eps)).to(residual.dtype)
        if next_gain is None:
            return None
        return self._norm(residual, next_gain, next_eps).to(self.dtype)

    def glu_clamped(self, gate_up, limit, slope, ff=None, shift=1.0):
        ff = ff or gate_up.shape[-1] // 2
        g = torch.clamp(gate_up[..., :ff].to(self.acc), max=limit)
        u = torch.clamp(gate_up[..., ff:2 * ff].to(self.acc), min=-limit, max=limit)
        return (g * torch.sigmoid(slope * g) * (u + shift)).to(self.dtype)

    # -- mixers with a state per row -------------------------------------------------------------
    @staticmethod
    def _sequences(ctx):
        starts = ctx.seq_qstart.cpu().tolist()
        rows = ctx.seq_rows.cpu().tolist()
        return [(rows[i], starts[i], starts[i + 1]) for i in range(len(rows))]

    def token_shift(self, h, mu, state, offset, ctx):
        N, d = h.shape
        hf = h.to(self.acc)
        prev = torch.empty_like(hf)
        for row, lo, hi in self._sequences(ctx):
            prev[lo] = state[row, offset:offset + d].to(self.acc)
            prev[lo + 1:hi] = hf[lo:hi - 1]
            state[row, offset:offset + d] = hf[hi - 1].to(state.dtype)
        return (hf.unsqueeze(0) + (prev - hf).unsqueeze(0) * mu.to(self.acc).unsqueeze(1)).to(self.dtype)

    def wkv_decay(self, t, w2_t, w0):
        z = torch.tanh(t.to(self.acc)) @ w2_t.to(self.acc) + w0.to(self.acc)
        return torch.exp(-torch.exp(z)).to(torch.float32 if self.acc == torch.float32 else self.acc)

    def wkv(self, r, k, v, decay, g, bonus, gain, eps, H, state, offset, ctx):
        N, C = r.shape
        D = C // H
        A = self.acc
        r, k, v, decay, g = (t.to(A).view(N, H, D) for t in (r, k, v, decay, g))
        out = torch.empty((N, H, D), dtype=A, device=r.device)
        for row, lo, hi in self._sequences(ctx):
            S = state[row, offset:offset + H * D * D].to(A).view(H, D, D).clone()
            for t in range(lo, hi):
                kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
                out[t] = torch.einsum("hk,hkv->hv", r[t], S + bonus.to(A).unsqueeze(-1) * kv)
                S = decay[t].unsqueeze(-1) * S + kv
            state[row, offset:offset + H * D * D] = S.reshape(-1).to(state.dtype)
        out = out / torch.sqrt(out.pow(2).mean(-1, keepdim=True) + eps)
        out = out * gain.to(A).view(H, D) * (g * torch.sigmoid(g))
        return out.reshape(N, C).to(self.dtype)

    def causal_conv_silu(self, x, col, C, weight, bias, state, offset, ctx):
        taps = weight.shape[1]
        A = self.acc
        xin = x[:, col:col + C].to(A)
        out = torch.empty((x.shape[0], C), dtype=A, device=x.device)
        for row, lo, hi in self._sequences(ctx):
            before = state[row, offset:offset + (taps - 1) * C].to(A).view(taps - 1, C)
            seq = torch.cat([before, xin[lo:hi]], dim=0)
            n = hi - lo
            y = bias.to(A).expand(n, -1).clone()
            for j in range(taps):
                y = y + seq[j:j + n] * weight[:, j].to(A)
            out[lo:hi] = y
            if taps > 1:
                state[row, offset:offset + (taps - 1) * C] = seq[n:].reshape(-1).to(state.dtype)
        return (out * torch.sigmoid(out)).to(self.dtype)

    def ssd(self, xbc, dt, dt_bias, a_log, skip, H, P, Ns, G, state, offset, ctx):
        A = self.acc
        N = xbc.shape[0]
        inner = H * P
        x = xbc[:, :inner].to(A).view(N, H, P)
        B = xbc[:, inner:inner + G * Ns].to(A).view(N, G, Ns).repeat_interleave(H // G, dim=1)
        Cm = xbc[:, inner + G * Ns:].to(A).view(N, G, Ns).repeat_interleave(H // G, dim=1)
        dt = torch.nn.functional.softplus(dt.to(A) + dt_bias.to(A), threshold=30.0)
        rate = torch.exp(a_log.to(A))
        out = torch.empty((N, H, P), dtype=A, device=xbc.device)
        for row, lo, hi in self._sequences(ctx):
            S = state[row, offset:offset + H * Ns * P].to(A).view(H, Ns, P).clone()
            for t in range(lo, hi):
                S = torch.exp(-rate * dt[t]).view(H, 1, 1) * S + (dt[t].unsqueeze(-1) * B[t]).unsqueeze(-1) * x[t].unsqueeze(-2)
                out[t] = torch.einsum("hn,hnp->hp", Cm[t], S) + skip.to(A).unsqueeze(-1) * x[t]
            state[row, offset:offset + H * Ns * P] = S.reshape(-1).to(state.dtype)
        return out.reshape(N, inner).to(torch.float32 if A == torch.float32 else A)

    def gated_group_norm(self, y, z, gain, groups, eps, gate_first=True, sigmoid=False):
        A = self.acc
        N, inner = y.shape
        zz = z[:, :inner].to(A)
        gate = torch.sigmoid(zz) if sigmoid else zz * torch.sigmoid(zz)
        y = y.to(A) * gate if gate_first else y.to(A)
        y = y.view(N, groups, inner // groups)
        y = y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps)
        y = y.reshape(N, inner) * gain.to(A)
        return (y if gate_first else y * gate).to(self.dtype)

    # -- attention over a cached latent ------------------------------------------------------------
    def _turn_pairs(self, x, positions, inv_freq, magnitude=1.0):
        """Pairs (2i, 2i + 1) of the first 2 * len(inv_freq) elements of the last axis; x [N, ..., D]."""
        dims = 2 * inv_freq.numel()
        ang = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
        shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
        cos, sin = (ang.cos().to(self.acc) * magnitude).view(shape), (ang.sin().to(self.acc) * magnitude).view(shape)
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out = x.clone()
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
        return out

    def rmsnorm_cols(self, x, weight, eps):
        return self._norm(x, weight, eps).to(self.dtype)

    def latent_write(self, kvd, R, Dr, gain, eps, inv_freq, positions, token_rows, slot):
        A = self.acc
        latent = self._norm(kvd[:, :R], gain, eps)
        shared = self._turn_pairs(kvd[:, R:R + Dr].to(A), positions, inv_freq)
        bs = slot.block_size
        pos = positions.long()
        page = slot.block_table[token_rows.long(), pos // bs].long()
        row = torch.zeros((kvd.shape[0], slot.k.shape[-1]), dtype=A, device=kvd.device)
        row[:, :R], row[:, R:R + Dr] = latent, shared
        slot.k[page, 0, pos % bs] = row.to(slot.k.dtype)

    def latent_query(self, q, H, D, Dr, w_uk_t, width, inv_freq, positions):
        A = self.acc
        N = q.shape[0]
        R = w_uk_t.shape[1]
        q = q.to(A).view(N, H, D + Dr)
        out = torch.zeros((N, H, width), dtype=A, device=q.device)
        out[..., :R] = torch.einsum("nhd,hrd->nhr", q[..., :D], w_uk_t.to(A))
        out[..., R:R + Dr] = self._turn_pairs(q[..., D:], positions, inv_freq)
        return out.to(self.dtype)

    def head_project(self, x, w):
        H, n_out, K = w.shape
        y = torch.einsum("nhk,hok->nho", x[..., :K].to(self.acc), w.to(self.acc))
        return y.reshape(x.shape[0], H * n_out).to(self.dtype)

    # -- attention whose keys and values differ in size, retention, routed experts, side input --------
    def attn_prepare(self, x, cols, Hq, Hkv, D, Dv, P, q_gain, k_gain, eps, inv_freq, rotary_dim, positions,
                     token_rows, slot, first=None, lam=None):
        A = self.acc
        N = x.shape[0]
        cq, ck, cv = cols
        q = x[:, cq:cq + Hq * D].reshape(N, Hq, D).to(A)
        k = x[:, ck:ck + Hkv * D].reshape(N, Hkv, D).to(A)
        if q_gain is not None:
            q, k = self._norm(q, q_gain, eps), self._norm(k, k_gain, eps)
        if rotary_dim:
            q = self._rotate(q, positions, inv_freq, rotary_dim)
            if Hkv:
                k = self._rotate(k, positions, inv_freq, rotary_dim)
        out = torch.zeros((N, Hq, P), dtype=self.dtype, device=x.device)
        out[..., :D] = q.to(self.dtype)
        if slot is not None and Hkv:
            v = x[:, cv:cv + Hkv * Dv].to(A)
            if first is not None:
                l = lam.to(A).reshape(())
                v = (1.0 - l) * v + l * first.to(A)
            kp = torch.zeros((N, Hkv, P), dtype=slot.k.dtype, device=x.device)
            vp = torch.zeros((N, Hkv, P), dtype=slot.v.dtype, device=x.device)
            kp[..., :D] = k.to(slot.k.dtype)
            vp[..., :Dv] = v.reshape(N, Hkv, Dv).to(slot.v.dtype)
            self.kv_write(kp, vp, positions, token_rows, slot)
        return out

    def head_gate(self, o, H, P, Dv, gate):
        N = o.shape[0]
        y = o.view(N, H, P)[..., :Dv].to(self.acc)
        if gate is not None:
            y = y * torch.sigmoid(gate.to(self.acc)).unsqueeze(-1)
        return y.reshape(N, H * Dv).to(self.dtype)

    def retention(self, x, cols, H, D, Dv, inv_freq, rotary_dim, k_scale, decays, state, offset, ctx):
        A = self.acc
        N = x.shape[0]
        cq, ck, cv = cols
        q = x[:, cq:cq + H * D].reshape(N, H, D).to(A)
        k = x[:, ck:ck + H * D].reshape(N, H, D).to(A)
        v = x[:, cv:cv + H * Dv].reshape(N, H, Dv).to(A)
        if rotary_dim:
            q = self._rotate(q, ctx.positions, inv_freq, rotary_dim)
            k = self._rotate(k, ctx.positions, inv_freq, rotary_dim)
        k = k * k_scale
        out = torch.empty((N, H, Dv), dtype=A, device=x.device)
        for row, lo, hi in self._sequences(ctx):
            S = state[row, offset:offset + H * D * Dv].to(A).view(H, D, Dv).clone()
            for t in range(lo, hi):
                S = decays.to(A).view(H, 1, 1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
                out[t] = torch.einsum("hk,hkv->hv", q[t], S)
            state[row, offset:offset + H * D * Dv] = S.reshape(-1).to(state.dtype)
        return out.reshape(N, H * Dv).to(torch.float32 if A == torch.float32 else A)

    def relu_squared(self, x):
        return (torch.relu(x.to(self.acc)) ** 2).to(self.dtype)

    def moe_route(self, logits, correction, top, n_groups=1, keep_groups=1, renorm_eps=1e-20, scoring="softmax",
                  group_top=1, scale=1.0):
        A = self.acc
        s = torch.softmax(logits.to(A), dim=-1) if scoring == "softmax" else torch.sigmoid(logits.to(A))
        c = s if correction is None else s + correction.to(A)
        N, E = s.shape
        if n_groups > 1 and keep_groups < n_groups:
            per = E // n_groups
            best = c.view(N, n_groups, per).sort(-1, descending=True).values[..., :group_top].sum(-1)
            kept = torch.zeros((N, n_groups), dtype=torch.bool, device=s.device)
            for _ in range(keep_groups):                      # the lower index among equals
                g = torch.where(kept, torch.full_like(best, -float("inf")), best).argmax(-1)
                kept[torch.arange(N), g] = True
            c = torch.where(kept.repeat_interleave(per, dim=1), c, torch.full_like(c, -float("inf")))
        idx = torch.empty((N, top), dtype=torch.int64, device=s.device)
        taken = torch.zeros_like(c, dtype=torch.bool)
        for r in range(top):
            e = torch.where(taken, torch.full_like(c, -float("inf")), c)
            # argmax returns the first of equal maxima only by convention; make it so
            m = e.max(-1, keepdim=True).values
            first = (e == m).to(torch.int64).argmax(-1)
            idx[:, r] = first
            taken[torch.arange(N), first] = True
        w = torch.gather(s, 1, idx)
        w = w / (w.sum(-1, keepdim=True) + renorm_eps) * scale
        return idx.to(torch.int32), w.to(torch.float32 if A == torch.float32 else A)

    def moe_experts(self, x, idx, weight, w_gate_up, w_down, limit, slope, extra=None, shift=1.0, extra_gate=None):
        A = self.acc
        N, top = idx.shape
        ff = w_gate_up.shape[1] // 2
        out = torch.zeros((N, w_down.shape[1]), dtype=A, device=x.device)
        if extra is not None:
            out += extra.to(A) if extra_gate is None else extra.to(A) * torch.sigmoid(extra_gate.to(A)).unsqueeze(-1)
        for r in range(top):
            e = idx[:, r].long()
            both = torch.einsum("nk,nok->no", x.to(A), w_gate_up[e].to(A)).to(self.dtype)
            act = self.glu_clamped(both, limit, slope, ff, shift)
            y = torch.einsum("nk,nok->no", act.to(A), w_down[e].to(A))
            out += weight[:, r:r + 1].to(A) * y
        return out.to(torch.float32 if A == torch.float32 else A)

    def side_gate(self, t, table, col0, token_ids):
        z = t.to(self.acc)
        g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        e = table[token_ids.long(), col0:col0 + t.shape[1]].to(self.acc)
        return (g * e).to(self.dtype)

    def add_cast(self, residual, delta):
        if delta is not None:
            residual += (delta.sum(0) if delta.dim() == 3 else delta).to(residual.dtype)
        return residual.to(self.dtype)

    # -- norms on results with a weighted sum over depth; window attention with pooled blocks; linear attention ----
    def depth_begin(self, residual, total, cast=False):
        kept = torch.zeros((total,) + tuple(residual.shape), dtype=residual.dtype, device=residual.device)
        kept[0] = residual
        return (kept, residual.to(self.dtype)) if cast else kept

    def norm_add_cast(self, residual, y, gain, eps, cast=True, depth=None):
        residual += self._norm(y, gain, eps).to(residual.dtype)
        if depth is not None:
            return self.depth_average(residual, *depth, cast=cast)
        return residual.to(self.dtype) if cast else None

    def depth_average(self, residual, kept, count, weights, cast=True):
        kept[count] = residual
        w = weights.to(self.acc).view(-1, 1, 1)
        residual.copy_((w[:count + 1] * kept[:count + 1].to(self.acc)).sum(0).to(residual.dtype))
        return residual.to(self.dtype) if cast else None

    def window_prepare(self, x, cols, Hq, Hkv, D, Dv, P, bias, q_gain, k_gain, norm, eps, inv_freq, rotary_dim, value_freq,
                       positions, token_rows, slot, magnitude=1.0):
        A = self.acc
        N = x.shape[0]
        cq, ck, cv = cols
        q, k, v = x[:, cq:cq + Hq * D].to(A), x[:, ck:ck + Hkv * D].to(A), x[:, cv:cv + Hkv * Dv].to(A)
        if bias is not None:
            b = bias.to(A)
            q, k, v = q + b[cq:cq + Hq * D], k + b[ck:ck + Hkv * D], v + b[cv:cv + Hkv * Dv]
        if norm == "whole":
            q, k = self._norm(q, q_gain, eps), self._norm(k, k_gain, eps)
        q, k, v = q.reshape(N, Hq, D), k.reshape(N, Hkv, D), v.reshape(N, Hkv, Dv)
        if norm == "head":
            q, k = self._norm(q, q_gain, eps), self._norm(k, k_gain, eps)
        if rotary_dim:
            q = self._turn_pairs(q, positions, inv_freq, magnitude)
            k = self._turn_pairs(k, positions, inv_freq, magnitude)
        if norm == "turned":
            q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps)
            k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps)
        if value_freq is not None:
            v = self._turn_pairs(v, positions, value_freq)
        out = torch.zeros((N, Hq, P), dtype=self.dtype, device=x.device)
        out[..., :D] = q.to(self.dtype)
        if slot is None:
            return out
        kp = torch.zeros((N, Hkv, P), dtype=slot.k.dtype, device=x.device)
        vp = torch.zeros((N, Hkv, P), dtype=slot.v.dtype, device=x.device)
        kp[..., :D] = k.to(slot.k.dtype)
        vp[..., :Dv] = v.to(slot.v.dtype)
        self.kv_write(kp, vp, positions, token_rows, slot)
        return out

    def pool_blocks(self, slot, ctx):
        """The means of the blocks whose last position is one of the step's, from the pages."""
        per, bs, means = slot.pool, slot.block_size, slot.pooled
        table, mtable = slot.block_table.cpu().numpy(), means.block_table.cpu().numpy()
        ends = ctx.seq_ctx.cpu().tolist()
        for i, (row, lo, hi) in enumerate(self._sequences(ctx)):
            start = ends[i] - (hi - lo)
            for b in range(start // per, ends[i] // per):
                idx = np.arange(b * per, b * per + per)
                pages = torch.as_tensor(table[row, idx // bs].astype(np.int64))
                offs = torch.as_tensor(idx % bs)
                page = int(mtable[row, b // bs])
                means.k[page, :, b % bs] = slot.k[pages, :, offs].to(self.acc).mean(0).to(means.k.dtype)
                means.v[page, :, b % bs] = slot.v[pages, :, offs].to(self.acc).mean(0).to(means.v.dtype)

    def turn_back(self, o, H, P, Dv, value_freq, positions):
        N = o.shape[0]
        y = o.view(N, H, P)[..., :Dv].to(self.acc)
        if value_freq is not None:
            y = self._turn_pairs(y, -positions, value_freq)
        return y.reshape(N, H * Dv).to(self.dtype)

    def linear_attention(self, x, cols, H, D, Dv, q_scale, activate, decays, z, z_bias, tau, state, offset, ctx,
                         prepared=None, ones=0):
        A = self.acc
        N = x.shape[0]
        cq, ck, cv = cols
        q = x[:, cq:cq + H * D].reshape(N, H, D).to(A)
        k = x[:, ck:ck + H * D].reshape(N, H, D).to(A)
        v = x[:, cv:cv + H * (Dv - ones)].reshape(N, H, Dv - ones).to(A)
        if ones:
            v = torch.cat([v, torch.ones((N, H, ones), dtype=A, device=x.device)], dim=-1)
        if activate:
            q, k, v = q * torch.sigmoid(q), k * torch.sigmoid(k), v * torch.sigmoid(v)
        q = q * q_scale
        if prepared is not None:
            q, k, decay = (prepared[:, j].reshape(N, H, D).to(A) for j in range(3))
        elif z is not None:
            decay = torch.exp(torch.nn.functional.logsigmoid(z.to(A) + z_bias.to(A)) / tau).view(N, H, D)
        else:
            decay = decays.to(A).view(1, H, 1).expand(N, H, D)
        out = torch.empty((N, H, Dv), dtype=A, device=x.device)
        for row, lo, hi in self._sequences(ctx):
            S = state[row, offset:offset + H * D * Dv].to(A).view(H, D, Dv).clone()
            for t in range(lo, hi):
                S = decay[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
                out[t] = torch.einsum("hk,hkv->hv", q[t], S)
            state[row, offset:offset + H * D * Dv] = S.reshape(-1).to(state.dtype)
        return out.reshape(N, H * Dv).to(torch.float32 if A == torch.float32 else A)

    def memory_gates(self, gates, bias, cap, x, cols, H, D, q_scale, state, offset, ctx):
        A = self.acc
        N = x.shape[0]
        cq, ck, _ = cols
        g = cap * torch.tanh((gates.to(A) + bias.to(A)) / cap)
        gi, gf = g[:, :H], torch.nn.functional.logsigmoid(g[:, H:])
        q = x[:, cq:cq + H * D].reshape(N, H, D).to(A) * q_scale
        k = x[:, ck:ck + H * D].reshape(N, H, D).to(A)
        out_dtype = torch.float32 if A == torch.float32 else A
        prep = torch.empty((N, 3, H * D), dtype=out_dtype, device=x.device)
        maxima = torch.empty((N, H), dtype=out_dtype, device=x.device)
        for row, lo, hi in self._sequences(ctx):
            m = state[row, offset:offset + H].to(A).clone()
            for t in range(lo, hi):
                new = torch.maximum(gf[t] + m, gi[t])
                prep[t, 0] = q[t].reshape(-1).to(out_dtype)
                prep[t, 1] = (torch.exp(gi[t] - new).unsqueeze(-1) * k[t]).reshape(-1).to(out_dtype)
                prep[t, 2] = torch.exp(gf[t] + m - new).unsqueeze(-1).expand(H, D).reshape(-1).to(out_dtype)
                maxima[t] = new.to(out_dtype)
                m = new
            state[row, offset:offset + H] = m.to(state.dtype)
        return prep, maxima

    def memory_finish(self, raw, maxima, z, gain, H, Dv, eps, den_eps):
        A = self.acc
        N = raw.shape[0]
        r = raw.view(N, H, Dv + 1).to(A)
        den = torch.maximum(r[..., Dv].abs(), torch.exp(-maxima.to(A))) + den_eps
        o = r[..., :Dv] / den.unsqueeze(-1)
        o = o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        y = o.reshape(N, H * Dv) * gain.to(A) * torch.sigmoid(z[:, :H * Dv].to(A))
        return y.to(self.dtype)

    def diff_combine(self, o, H, G, P, Dv, lam, eps, out_scale):
        A = self.acc
        N = o.shape[0]
        a = o.view(N, G, 2, H // G, P)[..., :Dv].to(A)
        y = a[:, :, 0] - lam * a[:, :, 1]
        y = y / torch.sqrt(y.pow(2).mean(-1, keepdim=True) + eps) * out_scale
        return y.reshape(N, H * Dv).to(self.dtype)

    def scaled_sum(self, a, a_scale, b, b_scale, bias=None):
        y = a.to(self.acc)
        if bias is not None:
            y = y + bias.to(self.acc)
        y = a_scale * y
        if b is not None:
            y = y + b_scale * b.to(self.acc)
        return y.to(torch.float32 if self.acc == torch.float32 else self.acc)

    def glu_gelu(self, gate_up, ff):
        z = gate_up[..., :ff].to(self.acc)
        g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        return (g * gate_up[..., ff:2 * ff].to(self.acc)).to(self.dtype)

    # -- sampling ----------------------------------------------------------------------------
    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, temperature, seed, draws):
        """Greedy where temperature is 0; else the inverse-CDF draw of softmax(logits / T)
        at the uniform number of (seed, draw)."""
        out = []
        for i in range(logits.shape[0]):
            T = float(temperature[i])
            if T <= 0.0:
                out.append(int(logits[i].argmax()))
                continue
            u = uniform_of(int(seed[i]), int(draws[i]))
            p = torch.softmax(logits[i].double() / T, dim=-1)
            cdf = torch.cumsum(p, dim=-1)
            tok = int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=cdf.dtype, device=cdf.device), right=True))
            out.append(min(tok, logits.shape[1] - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
