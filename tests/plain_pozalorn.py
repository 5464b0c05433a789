"""Pozalorn the plain way: whole sequences in float64, no cache, no batches, one function per
mechanism, written from the design's equations. It shares no code with ``socrates_amd``; the
tests compare the framework with it.

A model is (config dict as config.json holds it, {tensor name: torch tensor}).
"""

import math

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims); with ``scaling`` (factor, low, high, original) a frequency whose wavelength
    is longer than original/low is divided by factor, one shorter than original/high stays, and between
    the two the result slides from the one to the other."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            wave = 2.0 * math.pi / f
            if wave < scaling["original"] / scaling["high"]:
                pass
            elif wave > scaling["original"] / scaling["low"]:
                f = f / scaling["factor"]
            else:
                s = (scaling["original"] / wave - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def turn_pairs(x, positions, dims, freq, sign=1.0):
    """x [T, H, D]: elements 2i and 2i + 1 (i < dims/2) are one pair, turned by sign * position * freq[i];
    elements from dims on pass."""
    a = sign * positions.to(F)[:, None] * freq[None, :]
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def linear_attention(q, k, v, decay):
    """S_t = diag(decay_t) S_(t-1) + k_t v_t^T (row i of a head's state is scaled by the decay of key channel i),
    o_t = S_t^T q_t. q, k [T, H, D], v [T, H, Dv], decay [T, H, D]."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=F)
    o = torch.empty(T, H, v.shape[-1], dtype=F)
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return o


def gla(h, W, m, eps):
    """Gated linear attention: a decay per key channel that depends on the token."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W["k"].T).view(T, H, D)
    v = (h @ W["v"].T).view(T, H, Dv)
    z = (h @ W["a1"].T) @ W["a2"].T + W["a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, D)
    o = rms(linear_attention(q, k, v, alpha), eps) * W["norm"]
    return (o.reshape(T, H * Dv) * silu(h @ W["g"].T)) @ W["o"].T


def lightning(h, W, m, eps):
    """Linear attention with a fixed decay per head over activated q, k, v; the heads are normed together."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W["q"].T).view(T, H, D)
    k = silu(h @ W["k"].T).view(T, H, D)
    v = silu(h @ W["v"].T).view(T, H, Dv)
    decay = torch.tensor(m["decay"], dtype=F)[None, :, None].expand(T, H, D)
    o = linear_attention(q, k, v, decay).reshape(T, H * Dv)
    return (rms(o, eps) * W["norm"] * torch.sigmoid(h @ W["g"].T)) @ W["o"].T


def projections(h, W, m):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ W["q"].T + W["q.b"]
    k = h @ W["k"].T + W["k.b"]
    v = (h @ W["v"].T + W["v.b"]).view(T, G, Dv)
    return q, k, v


def softmax_over(s, seen, sink=None):
    """Weights of the visible scores; ``sink`` (one number) joins the denominator and has no value."""
    s = torch.where(seen, s, torch.full_like(s, -math.inf))
    top = s.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.expand_as(top))
    e = torch.exp(s - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return e / total


def window_attention(h, W, m, eps):
    """Softmax attention over a window, q and k normed per head, a learned sink per head in the denominator."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q, k, v = projections(h, W, m)
    q = rms(q.view(T, H, D), eps) * W["q.norm"]
    k = rms(k.view(T, G, D), eps) * W["k.norm"]
    freq = frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q = turn_pairs(q, pos, m["rot"]["dims"], freq)
    k = turn_pairs(k, pos, m["rot"]["dims"], freq)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < m["mask"]["size"])
    out = torch.empty(T, H, Dv, dtype=F)
    for a in range(H):
        b = a // (H // G)
        p = softmax_over((q[:, a] @ k[:, b].T) * m["scale"], seen, W["sink"][a])
        out[:, a] = p @ v[:, b]
    return out.reshape(T, H * Dv) @ W["o"].T + W["o.b"]


def pooled_attention(h, W, m, eps):
    """Softmax attention over a window and, before it, one mean key and value per block of tokens that
    ends before the window begins; q and k normed over the whole projection; values turned by their
    position and the result turned back by the query's."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, P = m["mask"]["size"], m["mask"]["pool"]
    pos = torch.arange(T)
    q, k, v = projections(h, W, m)
    q = (rms(q, eps) * W["q.norm"]).view(T, H, D)
    k = (rms(k, eps) * W["k.norm"]).view(T, G, D)
    freq = frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q = turn_pairs(q, pos, m["rot"]["dims"], freq)
    k = turn_pairs(k, pos, m["rot"]["dims"], freq)
    vfreq = frequencies(Dv, m["rot"]["base"])
    v = turn_pairs(v, pos, Dv, vfreq)
    B = T // P
    kb = k[:B * P].view(B, P, G, D).mean(1)
    vb = v[:B * P].view(B, P, G, Dv).mean(1)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < size)
    last = torch.arange(B)[None, :] * P + P - 1
    seen = torch.cat([seen, last <= i - size], dim=1)
    out = torch.empty(T, H, Dv, dtype=F)
    for a in range(H):
        b = a // (H // G)
        keys = torch.cat([k[:, b], kb[:, b]], dim=0)
        values = torch.cat([v[:, b], vb[:, b]], dim=0)
        p = softmax_over((q[:, a] @ keys.T) * m["scale"], seen)
        out[:, a] = p @ values
    out = turn_pairs(out, pos, Dv, vfreq, sign=-1.0)
    return out.reshape(T, H * Dv) @ W["o"].T


def parallel(h, W, m, eps):
    left = window_attention(h, sub(W, "left."), m["left"], eps)
    right = lightning(h, sub(W, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense(h, W):
    return (gelu_tanh(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F) for k, v in tensors.items() if k.startswith(prefix)}


MIXERS = {"gla": gla, "attention": pooled_attention, "parallel": parallel}


def forward(cfg, tensors, tokens, return_layers=False):
    """float64 logits [T, vocab] of the whole sequence (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = tensors["embed"].to(F)[torch.as_tensor(tokens, dtype=torch.long)]
    results = [x]                                          # X_0, then every layer's own result
    after = []
    for i, layer in enumerate(cfg["layers"]):
        W = sub(tensors, f"l{i}.")
        x = x + rms(MIXERS[layer["type"]](x, sub(W, "mix."), layer["mixer"], eps), eps) * W["norm1"]
        if layer.get("mlp") is not None:
            x = x + rms(dense(x, sub(W, "mlp.")), eps) * W["norm2"]
        results.append(x)
        x = sum(W["dwa"][j] * results[j] for j in range(i + 2))
        after.append(x)
    logits = (rms(x, eps) * tensors["final.norm"].to(F)) @ tensors["head"].to(F).T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy(cfg, tensors, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(cfg, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
