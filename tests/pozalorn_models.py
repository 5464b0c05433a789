"""Small Pozalorn configurations and seeded weights for the tests, and the checks that the CPU and the
GPU tests share. Sizes differ from model to model in everything that can differ: layer order, head
counts and groups, key and value sizes (equal and unequal, also none a multiple of 16), rotations over
part of a head or all of it, with and without stretched frequencies, windows shorter and longer than a
block of pooled tokens, blocks that divide neither the window nor a page, decays, temperatures, the
scales of the two sides, layers without feed-forward."""

import json
import math
import random
from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

import plain_pozalorn as plain
from helpers import make_runner, replay
from mitisun_models import CUTS, compare, row_errors  # noqa: F401  (shared by the test files)


def rot(dims, base=10000.0, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def window(heads, kv_heads, dim, vdim, size, rotation, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
            "rot": rotation, "mask": {"size": size}}


def attention(heads, kv_heads, dim, vdim, size, pool, rotation, scale=None):
    m = window(heads, kv_heads, dim, vdim, size, rotation, scale)
    m["mask"]["pool"] = pool
    return {"type": "attention", "mixer": m}


def lightning(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def parallel(left, right, left_scale=1.0, right_scale=1.0):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def gla(heads, dim, vdim, tau, rank=6):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "rank": rank}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def model(width, vocab, layers, mlps, eps=1e-5):
    """(config as config.json holds it, the ranks of the decays' inner projections by layer: only the
    tensors' shapes say them)."""
    out, ranks = [], {}
    for i, (layer, mlp) in enumerate(zip(layers, mlps)):
        layer = json.loads(json.dumps(layer))
        if "rank" in layer:
            ranks[i] = layer.pop("rank")
        layer["mlp"] = mlp
        out.append(layer)
    return {"architecture": "Pozalorn", "vocab": vocab, "width": width, "layers": out, "norm": {"eps": eps}}, ranks


STRETCH = (4.0, 1.0, 4.0, 64)           # wavelengths of 16 to 64 positions slide, longer ones are divided by 4
ONE_GLA = model(40, 61, [gla(3, 12, 20, 8.0, rank=5)], [dense(56)])
ONE_POOLED = model(48, 53, [attention(4, 2, 24, 12, size=7, pool=3, rotation=rot(8, 1000.0, STRETCH), scale=0.3)], [dense(40)], eps=1e-6)
ONE_PARALLEL = model(56, 67, [parallel(window(6, 3, 8, 20, 9, rot(8, 500.0)), lightning(2, 12, 16, (0.9, 0.99)), 0.6, 1.3)], [None])
MIX_A = model(64, 97, [gla(2, 16, 32, 12.0, rank=4),
                       attention(3, 1, 32, 16, size=9, pool=4, rotation=rot(16, 300000.0, (6.0, 1.0, 4.0, 32)), scale=0.2),
                       parallel(window(4, 2, 16, 24, 5, rot(16, 10000.0, STRETCH), scale=0.4), lightning(3, 8, 8, (0.5, 0.97, 1.0)), 0.7, 1.2),
                       attention(2, 2, 40, 24, size=12, pool=16, rotation=rot(20), scale=0.15),
                       gla(4, 8, 8, 1.0, rank=9)],
              [dense(80), None, dense(48), dense(100), None])
MIX_B = model(96, 130, [parallel(window(8, 2, 16, 16, 200, rot(16, 300000.0)), lightning(1, 48, 80, (0.98,)), 1.0, 1.0),
                        attention(6, 2, 48, 16, size=33, pool=5, rotation=rot(24, 100.0, (2.0, 1.0, 8.0, 128)), scale=0.1),
                        gla(1, 48, 80, 4.0, rank=16),
                        parallel(window(3, 3, 32, 8, 17, rot(4, 40000.0, STRETCH), scale=0.25), lightning(5, 4, 12, (0.6, 0.8, 0.9, 0.95, 0.999)), 1.5, 0.4)],
              [dense(200), dense(24), None, dense(64)], eps=3e-6)
MODELS = {"gla": ONE_GLA, "pooled": ONE_POOLED, "parallel": ONE_PARALLEL, "A": MIX_A, "B": MIX_B}
BLOCK = {"gla": 16, "pooled": 4, "parallel": 4, "A": 4, "B": 16}


def drawn_model(seed):
    """A configuration drawn from everything config.json can say: 2 to 5 layers in any order, sizes that are no
    multiples of anything (and sometimes 1), windows of one token up to longer than the prompts, blocks of one token
    up to longer than the window, layers without feed-forward."""
    rng = random.Random(seed)
    width = rng.choice([24, 36, 40, 50, 56, 64, 88, 128])

    def a_rotation(dim):
        dims = rng.choice([r for r in (2, 4, 8, 12, 16, 24, 40, 64) if r <= dim])
        scaling = None if rng.random() < 0.3 else (rng.choice([2.0, 4.0, 8.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([16, 64, 2048]))
        return rot(dims, rng.choice([100.0, 10000.0, 1e6]), scaling)

    def a_window(pooled):
        kv = rng.randint(1, 3)
        dim = rng.choice([4, 8, 12, 16, 24, 40, 64])
        vdim = rng.choice([4, 8, 20, 32, 48])
        return window(kv * rng.randint(1, 3), kv, dim, vdim, rng.choice([1, 2, 5, 17, 64] if pooled else [1, 2, 5, 17, 64, 300]),
                      a_rotation(dim), scale=rng.choice([0.1, 0.3, 1.0]) * 2 / dim ** 0.5)

    layers, mlps = [], []
    for _ in range(rng.randint(2, 5)):
        kind = rng.random()
        if kind < 0.35:
            layers.append(gla(rng.randint(1, 4), rng.choice([4, 8, 12, 16, 24, 40, 64]), rng.choice([4, 8, 20, 32, 48]),
                              rng.choice([1.0, 4.0, 16.0]), rank=rng.choice([1, 3, 8, 16])))
        elif kind < 0.65:
            m = a_window(True)
            m["mask"]["pool"] = rng.choice([1, 2, 3, 7, 16, 40])
            layers.append({"type": "attention", "mixer": m})
        else:
            heads = rng.randint(1, 4)
            layers.append(parallel(a_window(False), lightning(heads, rng.choice([4, 8, 12, 16, 24, 40, 64]), rng.choice([4, 8, 20, 32, 48]),
                                                              [rng.choice([0.5, 0.9, 0.97, 0.995, 1.0]) for _ in range(heads)]),
                                   rng.choice([0.5, 1.0, 1.4]), rng.choice([0.5, 1.0, 1.4])))
        mlps.append(None if rng.random() < 0.2 else dense(rng.choice([24, 50, 96])))
    return model(width, rng.choice([37, 64, 101]), layers, mlps, eps=rng.choice([1e-6, 1e-5, 1e-3]))


def tensor_shapes(made):
    cfg, ranks = made
    d, L = cfg["width"], len(cfg["layers"])
    t = {"embed": (cfg["vocab"], d), "head": (cfg["vocab"], d), "final.norm": (d,)}

    def linear(p, m, gate_norm):
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        t.update({p + "q": (H * D, d), p + "k": (H * D, d), p + "v": (H * Dv, d), p + "g": (H * Dv, d), p + "o": (d, H * Dv),
                  p + "norm": (gate_norm,)})

    def softmax(p, m, pooled):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t.update({p + "q": (H * D, d), p + "k": (G * D, d), p + "v": (G * Dv, d), p + "o": (d, H * Dv),
                  p + "q.b": (H * D,), p + "k.b": (G * D,), p + "v.b": (G * Dv,)})
        if pooled:
            t.update({p + "q.norm": (H * D,), p + "k.norm": (G * D,)})
        else:
            t.update({p + "q.norm": (D,), p + "k.norm": (D,), p + "o.b": (d,), p + "sink": (H,)})

    for i, layer in enumerate(cfg["layers"]):
        P, m, mlp = f"l{i}.", layer["mixer"], layer["mlp"]
        t[P + "norm1"] = (d,)
        t[P + "dwa"] = (i + 2,)
        p = P + "mix."
        if layer["type"] == "gla":
            linear(p, m, m["vdim"])
            r = ranks[i]
            t.update({p + "a1": (r, d), p + "a2": (m["heads"] * m["dim"], r), p + "a2.b": (m["heads"] * m["dim"],)})
        elif layer["type"] == "attention":
            softmax(p, m, True)
        else:
            softmax(p + "left.", m["left"], False)
            linear(p + "right.", m["right"], m["right"]["heads"] * m["right"]["vdim"])
        if mlp is not None:
            t[P + "norm2"] = (d,)
            t.update({P + "mlp.gate": (mlp["ff"], d), P + "mlp.up": (mlp["ff"], d), P + "mlp.down": (d, mlp["ff"])})
    return t


def random_weights(made, seed):
    """Weights in float32 that already hold bfloat16 values. Matrices are scaled so that every branch has results
    of order one; biases, sinks and the decays' logits are of order one and of both signs; the weights over depth
    are near an even share, of both signs here and there."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(made).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm", "norm1", "norm2"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "dwa":
            t = (1.0 + 0.5 * torch.randn(shape, generator=g)) * (2.0 / shape[0])
        elif name.endswith("a2.b"):
            t = 2.0 + 1.5 * torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "sink":
            t = torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_model(folder, made, seed, weights=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    weights = weights if weights is not None else random_weights(made, seed)
    (folder / "config.json").write_text(json.dumps(made[0]))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, str(folder / "model.safetensors"))
    return folder


def read_folder(folder):
    folder = Path(folder)
    return json.loads((folder / "config.json").read_text()), {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}


def oracle(folder, prompts):
    cfg, w = read_folder(folder)
    return [plain.forward(cfg, w, p).float() for p in prompts]


def check_trace(folder, ops, prompts, steps, tol, want=None, max_rows=4, block_size=16, num_blocks=None, max_len=512, what="",
                graphs=0):
    """Replay ``steps`` through the framework's step function and compare every position with the oracle."""
    runner = make_runner(folder, ops, max_rows=max_rows, max_len=max_len, block_size=block_size, num_blocks=num_blocks)
    if graphs:
        runner.enable_graphs(graphs)
    got = replay(runner, steps)
    want = want or oracle(folder, prompts)
    for i, p in enumerate(prompts):
        compare(got[f"r{i}"], want[i], tol, f"{what} request {i}")
    assert runner.cache.open_rows == []
    return runner
