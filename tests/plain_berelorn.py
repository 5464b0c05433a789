"""A plain, slow implementation of Berelorn: whole sequences in float64, no cache, one function per
mechanism, written from the equations and sharing no code with the package.

Notation: h [T, d] is a sublayer's input, W a dict of float64 tensors by their local names, positions
count from 0. ``rms(x)`` is x / sqrt(mean(x^2) + eps) over the last dimension.
"""

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotation_constants(rot):
    """(frequencies [dims / 2], magnitude) of a rotation over interleaved pairs, with the stretch that
    ``rot['scaling']`` = {factor, original, fast, slow} asks for: a pair index below ``lo`` keeps its frequency, one
    above ``hi`` has it divided by factor, a linear ramp in the index between them; cosines and sines are
    multiplied by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(index_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, rot):
    """x [T, ..., D]: elements 2i and 2i + 1 of the first rot.dims are turned by position * f_i."""
    if not rot or not rot.get("dims"):
        return x
    f, mag = rotation_constants(rot)
    dims = rot["dims"]
    ang = positions.to(F64)[:, None] * torch.tensor(f, dtype=F64)[None, :]            # [T, dims / 2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(T, mask):
    """[T, T] bool: query i sees key j <= i within the window, or among the kept first keys."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if mask:
        ok = ok & ((i - j < mask["size"]) | (j < mask.get("keep_first", 0)))
    return ok


def softmax_attention(q, k, v, scale, ok, softcap=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; query head h reads kv head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~ok, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def mlstm(h, W, m, eps, first_max=0.0):
    """Matrix memory with exponential gates held stable by a running maximum that starts at ``first_max`` (0)."""
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ W["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W["k"].T).view(T, H, D)
    v = (h @ W["v"].T).view(T, H, Dv)
    gi = cap * torch.tanh((h @ W["i"].T + W["i.b"]) / cap)                               # [T, H], a logarithm
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W["f"].T + W["f.b"]) / cap))
    out = torch.zeros(T, H, Dv, dtype=F64)
    for a in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        n = torch.zeros(D, dtype=F64)
        mx = first_max
        for t in range(T):
            new = max(float(gf[t, a]) + mx, float(gi[t, a]))
            keep, take = math.exp(float(gf[t, a]) + mx - new), math.exp(float(gi[t, a]) - new)
            S = keep * S + take * torch.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            mx = new
            den = max(abs(float(n @ q[t, a])), math.exp(-mx)) + 1e-6
            out[t, a] = (S.T @ q[t, a]) / den
    y = rms(out, eps).reshape(T, H * Dv) * W["norm"] * torch.sigmoid(h @ W["g"].T)
    return y @ W["o"].T


def differential_attention(h, W, m, eps, positions, borrowed=None):
    """Two softmax maps per head over the same values, the second subtracted with one weight for the layer.
    ``borrowed``: (keys after rotation, values) of the layer whose cache this one reads. Returns (result,
    (keys after rotation, values))."""
    T = h.shape[0]
    H, G, D, Dv, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["diff"])
    q = (h @ W["q"].T + W["q.b"]).view(T, H, 2, D)
    q = rotate_pairs(q, positions, m.get("rot"))
    if borrowed is None:
        k = (h @ W["k"].T + W["k.b"]).view(T, G, 2, D)
        k = rotate_pairs(k, positions, m.get("rot"))
        v = (h @ W["v"].T + W["v.b"]).view(T, G, Dv)
    else:
        k, v = borrowed
    ok = visible(T, m.get("mask"))
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, float(m["scale"]), ok)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, float(m["scale"]), ok)
    lam = math.exp(float((W["lq1"] * W["lk1"]).sum())) - math.exp(float((W["lq2"] * W["lk2"]).sum())) + diff
    o = rms(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * Dv) @ W["o"].T + W["o.b"], (k, v)


def keyed_attention(h, W, m, eps, positions):
    """Causal attention whose values are the keys as projected; q and k turned, then divided by their root mean
    square per head; soft-capped scores; a sigmoid gate per head."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W["q"].T).view(T, H, D)
    k = (h @ W["k"].T).view(T, G, D)
    v = k
    q = rms(rotate_pairs(q, positions, m.get("rot")), eps)
    k = rms(rotate_pairs(k, positions, m.get("rot")), eps)
    o = softmax_attention(q, k, v, float(m["scale"]), visible(T, None), softcap=m.get("softcap"))
    o = o * torch.sigmoid(h @ W["g"].T)[:, :, None]
    return o.reshape(T, H * v.shape[2]) @ W["o"].T


def choose_experts(s, top, count, keep):
    """s [E] scores of one token -> the chosen experts: the ``top`` largest among the ``keep`` groups (of ``count``
    equal groups of neighbours) whose two largest scores sum highest; the lower index among equals."""
    E = s.shape[0]
    size = E // count
    score = []
    for g in range(count):
        part = sorted((float(x) for x in s[g * size:(g + 1) * size]), reverse=True)
        score.append(sum(part[:2]))
    groups = sorted(range(count), key=lambda g: (-score[g], g))[:keep]
    allowed = [e for e in range(E) if e // size in groups]
    return sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]


def glu(h, W, prefix):
    g = h @ W[prefix + "gate"].T
    return (g * torch.sigmoid(g) * (h @ W[prefix + "up"].T)) @ W[prefix + "down"].T


def mixture(h, W, mlp):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.sigmoid(h @ W["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = choose_experts(s[t], r["top"], groups["count"], groups["keep"])
        total = sum(float(s[t, e]) for e in chosen) + 1e-20
        for e in chosen:
            out[t] += float(s[t, e]) / total * float(r.get("scale", 1.0)) * glu(h[t:t + 1], W, f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W["shared.sg"].T) * glu(h, W, "shared.")
    return out


def part(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, tokens, residuals=None, first_max=0.0):
    """Logits [T, vocab] of one sequence; ``residuals`` (a list) receives the stream after every layer.
    ``first_max``: where the running maxima of the matrix memories start (0 in the design; a test passes
    another value to show that it would see the difference)."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    x = W["embed"][tokens] * float((config.get("embedding") or {}).get("scale", 1.0))
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms(x, eps) * W[p + "norm1"]
        if layer["type"] == "mlstm":
            y = mlstm(h, part(W, p + "mix."), m, eps, first_max)
        elif layer["type"] == "attention":
            y, kept[i] = differential_attention(h, part(W, p + "mix."), m, eps, positions,
                                                kept[m["kv_from"]] if m.get("kv_from") is not None else None)
        elif layer["type"] == "attention_2":
            y = keyed_attention(h, part(W, p + "mix."), m, eps, positions)
        else:
            raise ValueError(layer["type"])
        x = x + rms(y, eps) * W[p + "norm1b"]
        if layer.get("mlp") is not None:
            h = rms(x, eps) * W[p + "norm2"]
            x = x + rms(mixture(h, part(W, p + "mlp."), layer["mlp"]), eps) * W[p + "norm2b"]
        if residuals is not None:
            residuals.append(x.clone())
    x = rms(x, eps) * W["final.norm"]
    return x @ W["embed"].T


def greedy(config, weights, prompt, n_new):
    """The n_new tokens that follow ``prompt`` when the largest logit is taken every time (the lowest index
    among equals)."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        tok = int(forward(config, weights, ids)[-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
