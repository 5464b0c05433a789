"""Small Berelorn configurations and seeded weights for the tests, and the checks that the CPU and the GPU
tests share. Sizes differ from model to model in everything that can differ: layer order, head counts and
groups (one to three query heads per kv head), key and value sizes (equal and unequal, also none a multiple
of 16), rotations over part of a head or all of it with and without the ramp, windows of 5 to 200 with 0 to
12 kept first tokens (more than the window among them) or no mask at all, layers that read another layer's
cache behind a wider or a narrower mask, gate caps, soft caps, experts with and without groups and shared
expert, one expert per token and all of them, layers without feed-forward, embedding and router scales."""

import json
import math
import random
from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

import plain_berelorn as plain
from helpers import make_runner, replay
from mitisun_models import CUTS, compare, row_errors  # noqa: F401  (shared by the test files)


def rot(dims, base=10000.0, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def memory(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def differential(heads, kv_heads, dim, vdim, size, keep, rotation, diff, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "diff": diff, "rot": rotation, "mask": None if size is None else {"size": size, "keep_first": keep}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def keyed(heads, kv_heads, dim, rotation, scale=None, softcap=30.0):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                                             "scale": scale if scale is not None else 1.0, "softcap": softcap, "rot": rotation}}


def moe(experts, top, ff, count=1, keep=1, scale=1.0, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale,
                                                             "groups": {"count": count, "keep": keep}},
           "shared": None if shared is None else {"ff": shared}}
    return out


def model(width, vocab, layers, mlps, eps=1e-5, embedding=1.0):
    out = []
    for layer, mlp in zip(layers, mlps):
        layer = json.loads(json.dumps(layer))
        layer["mlp"] = mlp
        out.append(layer)
    return {"architecture": "Berelorn", "vocab": vocab, "width": width, "embedding": {"scale": embedding}, "layers": out,
            "norm": {"eps": eps}}


RAMP = (4.0, 64, 8.0, 1.0)              # pairs 0 to 2 of 8 dimensions over a base of 1000 slide, later ones are divided by 4
ONE_MEMORY = model(40, 61, [memory(3, 12, 20, 8.0)], [moe(6, 2, 24, count=3, keep=2, scale=2.0, shared=40)], embedding=3.0)
ONE_DIFF = model(48, 53, [differential(4, 2, 24, 12, size=7, keep=3, rotation=rot(8, 1000.0, RAMP), diff=0.3, scale=0.3)], [None],
                 eps=1e-6)
ONE_KEYED = model(56, 67, [keyed(6, 2, 8, rot(8, 500.0, (3.0, 32, 4.0, 0.5)), scale=3.0, softcap=4.0)], [moe(5, 1, 32)], embedding=0.5)
MIX_A = model(64, 97, [memory(2, 16, 32, 15.0),
                       differential(3, 1, 32, 16, size=9, keep=2, rotation=rot(16, 300000.0, (6.0, 32, 16.0, 2.0)), diff=0.8, scale=0.2),
                       keyed(4, 4, 16, rot(16, 10000.0, RAMP), scale=2.0, softcap=50.0),
                       differential(3, 1, 32, 16, size=20, keep=0, rotation=rot(16, 300000.0, (6.0, 32, 16.0, 2.0)), diff=0.2, scale=0.3,
                                    kv_from=1),
                       memory(4, 8, 8, 3.0)],
              [moe(8, 3, 16, count=4, keep=2, scale=0.7, shared=48), None, moe(4, 4, 24, count=4, keep=4, scale=1.5),
               moe(9, 2, 20, count=3, keep=1, shared=16), None], embedding=6.0)
MIX_B = model(96, 130, [differential(8, 2, 16, 16, size=200, keep=12, rotation=rot(16, 300000.0), diff=0.5, scale=0.25),
                        differential(8, 2, 16, 16, size=5, keep=12, rotation=rot(16, 300000.0), diff=0.1, scale=0.4, kv_from=0),
                        memory(1, 48, 80, 20.0),
                        keyed(3, 1, 40, rot(20, 100.0, (2.0, 128, 32.0, 1.0)), scale=1.2, softcap=8.0),
                        differential(2, 2, 40, 24, size=None, keep=0, rotation=rot(24, 40000.0, RAMP), diff=0.4, scale=0.15)],
              [moe(12, 3, 24, count=6, keep=3, scale=1.2, shared=64), moe(3, 2, 40, count=3, keep=2), None,
               moe(16, 4, 8, count=2, keep=1, scale=2.5, shared=24), moe(2, 1, 64)], eps=3e-6)
MODELS = {"memory": ONE_MEMORY, "diff": ONE_DIFF, "keyed": ONE_KEYED, "A": MIX_A, "B": MIX_B}
BLOCK = {"memory": 16, "diff": 4, "keyed": 4, "A": 4, "B": 16}


def drawn_model(seed):
    """A configuration drawn from everything config.json can say: 2 to 5 layers in any order, sizes that are no
    multiples of anything (and sometimes 1), windows of one token up to longer than the prompts, kept first tokens
    from none to more than the window, layers on another layer's cache, layers without feed-forward."""
    rng = random.Random(seed)
    width = rng.choice([24, 36, 40, 50, 56, 64, 88, 128])

    def a_rotation(dim):
        dims = rng.choice([r for r in (0, 2, 4, 8, 12, 16, 24, 40, 64) if r <= dim])
        if not dims:
            return None
        scaling = None if rng.random() < 0.3 else (rng.choice([3.0, 4.0, 8.0]), rng.choice([16, 64, 4096]), rng.choice([4.0, 16.0]),
                                                   rng.choice([0.5, 1.0, 2.0]))
        return rot(dims, rng.choice([100.0, 10000.0, 1e6]), scaling)

    def a_moe():
        count = rng.choice([1, 2, 3, 4])
        per = rng.choice([1, 2, 3, 5])
        keep = rng.randint(1, count)
        return moe(count * per, rng.randint(1, keep * per), rng.choice([8, 24, 50]), count, keep, rng.choice([0.5, 1.0, 2.5]),
                   rng.choice([None, 16, 40]))

    layers, mlps, writers = [], [], []
    for i in range(rng.randint(2, 5)):
        kind = rng.random()
        if kind < 0.3:
            layers.append(memory(rng.randint(1, 4), rng.choice([4, 8, 12, 16, 24, 40, 64]), rng.choice([4, 8, 20, 32, 48]),
                                 rng.choice([1.0, 8.0, 30.0])))
        elif kind < 0.7:
            size = rng.choice([1, 2, 5, 17, 64, 300, None])
            keep = 0 if size is None else rng.choice([0, 1, 3, 8, 20])
            if writers and rng.random() < 0.5:
                j = rng.choice(writers)
                m = layers[j]["mixer"]
                layers.append(differential(m["heads"], m["kv_heads"], m["dim"], m["vdim"], size, keep, m["rot"], rng.choice([0.1, 0.5, 0.9]),
                                           rng.choice([0.1, 0.3, 1.0]) * 2 / m["dim"] ** 0.5, kv_from=j))
            else:
                kv = rng.randint(1, 3)
                dim = rng.choice([4, 8, 12, 16, 24, 40, 64])
                layers.append(differential(kv * rng.randint(1, 3), kv, dim, rng.choice([4, 8, 20, 32, 48]), size, keep, a_rotation(dim),
                                           rng.choice([0.1, 0.5, 0.9]), rng.choice([0.1, 0.3, 1.0]) * 2 / dim ** 0.5))
                writers.append(i)
        else:
            kv = rng.randint(1, 3)
            dim = rng.choice([4, 8, 12, 16, 24, 40, 64])
            layers.append(keyed(kv * rng.randint(1, 3), kv, dim, a_rotation(dim), rng.choice([0.5, 1.0, 3.0]), rng.choice([None, 2.0, 30.0])))
        mlps.append(None if rng.random() < 0.2 else a_moe())
    return model(width, rng.choice([37, 64, 101]), layers, mlps, eps=rng.choice([1e-6, 1e-5, 1e-3]), embedding=rng.choice([1.0, 4.0, 11.0]))


def tensor_shapes(cfg):
    d = cfg["width"]
    t = {"embed": (cfg["vocab"], d), "final.norm": (d,)}
    for i, layer in enumerate(cfg["layers"]):
        P, m, mlp = f"l{i}.", layer["mixer"], layer["mlp"]
        t[P + "norm1"] = t[P + "norm1b"] = (d,)
        p = P + "mix."
        if layer["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            t.update({p + "q": (H * D, d), p + "k": (H * D, d), p + "v": (H * Dv, d), p + "g": (H * Dv, d), p + "o": (d, H * Dv),
                      p + "norm": (H * Dv,), p + "i": (H, d), p + "i.b": (H,), p + "f": (H, d), p + "f.b": (H,)})
        elif layer["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "q": (2 * H * D, d), p + "q.b": (2 * H * D,), p + "o": (d, H * Dv), p + "o.b": (d,),
                      p + "lq1": (D,), p + "lk1": (D,), p + "lq2": (D,), p + "lk2": (D,)})
            if m.get("kv_from") is None:
                t.update({p + "k": (2 * G * D, d), p + "k.b": (2 * G * D,), p + "v": (G * Dv, d), p + "v.b": (G * Dv,)})
        else:
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            t.update({p + "q": (H * D, d), p + "k": (G * D, d), p + "g": (H, d), p + "o": (d, H * D)})
        if mlp is not None:
            t[P + "norm2"] = t[P + "norm2b"] = (d,)
            q = P + "mlp."
            t[q + "router"] = (mlp["router"]["experts"], d)
            for e in range(mlp["router"]["experts"]):
                t.update({f"{q}e{e}.gate": (mlp["expert"]["ff"], d), f"{q}e{e}.up": (mlp["expert"]["ff"], d),
                          f"{q}e{e}.down": (d, mlp["expert"]["ff"])})
            if mlp.get("shared"):
                ff = mlp["shared"]["ff"]
                t.update({q + "shared.gate": (ff, d), q + "shared.up": (ff, d), q + "shared.down": (d, ff), q + "shared.sg": (1, d)})
    return t


def random_weights(cfg, seed):
    """Weights in float32 that already hold bfloat16 values. Matrices are scaled so that every branch has results
    of order one; biases and gate logits are of order one and of both signs; the forget gates lean open."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith("f.b"):
            t = 2.0 + 1.5 * torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.6 * torch.randn(shape, generator=g) / math.sqrt(shape[0]) ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "router":
            t = torch.randn(shape, generator=g) * (3.0 / math.sqrt(shape[-1]))
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_model(folder, cfg, seed, weights=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    weights = weights if weights is not None else random_weights(cfg, seed)
    (folder / "config.json").write_text(json.dumps(cfg))
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
