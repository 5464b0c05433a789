"""Berelorn through the framework's step function, cache manager and scheduler, on the CPU with the stand-in
kernels, against the plain implementation in ``plain_berelorn``: every mechanism alone and in mixtures; whole
prompts, token-by-token decoding, portions down to two tokens, mixed batches in a pool so small that pages and
state rows are used again; the edges of the windows and of the kept first tokens, in a layer's own cache and in
one it reads from another layer; the first tokens of the matrix memory; far tokens through a state and through
hundreds of keys; the choice of experts; the configuration and the weights' names."""

import json
import math

import pytest
import torch

import plain_berelorn as plain
from berelorn_models import (BLOCK, CUTS, MODELS, RAMP, check_trace, compare, differential, drawn_model, keyed, memory, model, moe,
                             oracle, random_weights, read_folder, rot, tensor_shapes, write_model)
from helpers import make_runner, random_prompts
from socrates_amd.config import ConfigError, load_config
from socrates_amd.config.berelorn import BerelornConfig
from socrates_amd.config.specs import PairRopeSpec
from socrates_amd.engine import StepEntry
from socrates_amd.parts import cache_needs, expected_tensors
from socrates_amd.parts.registry import PagedKV, RowState
from torch_kernels import TorchKernels

TOL = 2e-4          # float32 stand-in kernels against the float64 oracle, in units of the logits' spread


def ops32():
    return TorchKernels(torch.float32, "cpu")


def ops64():
    return TorchKernels(torch.float64, "cpu", acc=torch.float64)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("berelorn")
    return {name: write_model(base / name, cfg, seed=i + 1) for i, (name, cfg) in enumerate(MODELS.items())}


# ---- configuration, plan, names ---------------------------------------------------------------------
def test_plan_follows_the_configuration(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, BerelornConfig) and cfg.to_dict() == MODELS["A"]
    plan = cfg.plan()
    needs = cache_needs(plan)
    # the memory's state: per head 16 x (32 + 1), and one running maximum per head
    assert isinstance(needs[0], RowState) and needs[0].shape == (2 * 16 * 33 + 2,)
    # two maps per kv head; keys of 32 beside values of 16 share pools of 32; the slot holds what the wider of its two
    # readers sees (layer 3 reads it behind a window of 20 with no kept keys, layer 1 behind 9 with 2)
    assert needs[1] == PagedKV(2, 32, 20, 2)
    assert needs[2] == PagedKV(4, 16, None, 0) and needs[3] is None
    assert [(s.layer, s.cache, s.write) for s in plan.order] == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 1, False), (4, 4, True)]
    assert plan.head_name is None and plan.embedding_scale == 6.0
    assert set(plan.ignorable) == {"l1.norm2", "l1.norm2b", "l4.norm2", "l4.norm2b"}
    names = expected_tensors(plan)
    want = tensor_shapes(MODELS["A"])
    assert set(names) == set(want)
    assert all(names[n].fits(want[n]) for n in want), [n for n in want if not names[n].fits(want[n])]
    # a reader behind a narrower mask than the writer's, and a layer without a mask
    needs = cache_needs(load_config(folders["B"]).plan())
    assert needs[0] == PagedKV(4, 16, 200, 12) and needs[1] is None and needs[4] == PagedKV(4, 48, None, 0)


def test_configuration_errors():
    good = MODELS["A"]

    def broken(change):
        bad = json.loads(json.dumps(good))
        change(bad)
        return bad
    with pytest.raises(ConfigError, match="unknown type"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(ConfigError, match="rot.dims"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34)))
    with pytest.raises(ConfigError, match="kv heads"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][2]["mixer"].update(kv_heads=3)))
    with pytest.raises(ConfigError, match="lacks"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][0]["mixer"].pop("gate_cap")))
    with pytest.raises(ConfigError, match="lacks"):
        BerelornConfig.from_dict(broken(lambda c: c.pop("norm")))
    with pytest.raises(ConfigError, match="earlier layer"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][3]["mixer"].update(kv_from=4)))
    with pytest.raises(ConfigError, match="of its own"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][3]["mixer"].update(kv_from=2)))
    with pytest.raises(ConfigError, match="must equal"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][3]["mixer"].update(heads=2)))
    with pytest.raises(ConfigError, match="vdim equals dim"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][2]["mixer"].update(vdim=8)))
    with pytest.raises(ConfigError, match="not possible"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][3]["mlp"]["router"].update(top=4)))
    with pytest.raises(ConfigError, match="feed-forward"):
        BerelornConfig.from_dict(broken(lambda c: c["layers"][0]["mlp"].update(kind="dense")))


# ---- each mechanism of the stand-in kernel set against the plain function ---------------------------------
@pytest.mark.parametrize("dims,base,ramp", [(8, 1000.0, RAMP), (16, 300000.0, (6.0, 32, 16.0, 2.0)), (48, 40000.0, (3.0, 4096, 32.0, 1.0)),
                                            (8, 100.0, None), (2, 7.0, (3.0, 4, 2.0, 1.0)), (20, 100.0, (2.0, 128, 32.0, 1.0))])
def test_ramped_frequencies(dims, base, ramp):
    """Pairs below the ramp keep their frequency, those above have it divided, those on it slide; cosines and sines
    grow with the logarithm of the factor."""
    scaling = None if ramp is None else dict(zip(("factor", "original", "fast", "slow"), ramp))
    want, magnitude = plain.rotation_constants({"dims": dims, "base": base, "scaling": scaling})
    spec = PairRopeSpec(dims=dims, base=base, ramp=ramp)
    assert spec.frequencies() == pytest.approx(want, rel=1e-13) and spec.magnitude == pytest.approx(magnitude, rel=1e-15)
    if ramp is not None and dims >= 8:
        plainest = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
        ratio = [a / b for a, b in zip(want, plainest)]
        assert max(ratio) <= 1.0 and min(ratio) >= 1.0 / ramp[0] - 1e-12 and all(b <= a + 1e-12 for a, b in zip(ratio, ratio[1:]))
        assert magnitude == pytest.approx(0.1 * math.log(ramp[0]) + 1.0)
    if ramp == RAMP:
        assert [round(a / b, 6) for a, b in zip(want, [1000.0 ** (-i / 4) for i in range(4)])] == [1.0, 0.625, 0.25, 0.25]


def _ctx(lengths, rows, starts):
    from types import SimpleNamespace
    q = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lengths)]).to(torch.int32)
    trow = torch.cat([torch.full((n,), r) for r, n in zip(rows, lengths)]).to(torch.int32)
    return SimpleNamespace(n_seqs=len(lengths), n_tokens=int(q[-1]), seq_qstart=q, seq_rows=torch.tensor(rows, dtype=torch.int32),
                           positions=pos, token_rows=trow, max_q_len=max(lengths),
                           seq_ctx=torch.tensor([s + n for s, n in zip(starts, lengths)], dtype=torch.int32),
                           max_ctx_len=max(s + n for s, n in zip(starts, lengths)))


def test_matrix_memory_in_portions_equals_the_plain_recurrence():
    """One sequence of 23 tokens in portions of 9, 1, 2 and 11 beside another sequence, from the state that each
    portion left (matrix, sum of keys and running maximum): the plain function over the whole sequence, with gates
    that swing from shut to wide open, so that the maximum moves and the floor exp(-m) of the denominator bites."""
    g = torch.Generator().manual_seed(4)
    H, D, Dv, T, d, cap = 3, 5, 7, 23, 16, 6.0
    h = torch.randn(T, d, generator=g, dtype=torch.float64)
    other = torch.randn(T, d, generator=g, dtype=torch.float64)
    W = {n: torch.randn(s, generator=g, dtype=torch.float64) * 0.4 for n, s in
         (("q", (H * D, d)), ("k", (H * D, d)), ("v", (H * Dv, d)), ("g", (H * Dv, d)), ("i", (H, d)), ("f", (H, d)))}
    W["i"] *= 8
    W["f"] *= 8
    W.update({"i.b": torch.tensor([-3.0, 0.0, 2.0], dtype=torch.float64), "f.b": torch.tensor([4.0, 0.0, -1.0], dtype=torch.float64),
              "norm": torch.randn(H * Dv, generator=g, dtype=torch.float64), "o": torch.eye(H * Dv, dtype=torch.float64)})
    want = plain.mlstm(h, W, {"heads": H, "dim": D, "vdim": Dv, "gate_cap": cap}, 1e-5)
    ops = ops64()
    w_first = torch.cat([W["g"], W["q"], W["k"], W["v"]])
    cols = (H * Dv, H * Dv + H * D, H * Dv + 2 * H * D)
    state = torch.zeros(4, 2 + H * D * (Dv + 1) + H, dtype=torch.float64)
    got, t = [], 0
    for n in (9, 1, 2, 11):
        ctx = _ctx([n, n], [2, 0], [t, t])
        x = torch.cat([h[t:t + n], other[t:t + n]])
        first = x @ w_first.T
        gates = x @ torch.cat([W["i"], W["f"]]).T
        prep, maxima = ops.memory_gates(gates, torch.cat([W["i.b"], W["f.b"]]), cap, first, cols, H, D, D ** -0.5, state,
                                        2 + H * D * (Dv + 1), ctx)
        raw = ops.linear_attention(first, cols, H, D, Dv + 1, 1.0, False, None, None, None, 1.0, state, 2, ctx, prepared=prep, ones=1)
        got.append(ops.memory_finish(raw, maxima, first, W["norm"], H, Dv, 1e-5, 1e-6)[:n])
        t += n
    assert torch.allclose(torch.cat(got), want, atol=1e-11)
    assert float(state[:, :2].abs().max()) == 0.0 and float(state[1].abs().max()) == 0.0
    assert float(state[2, -H:].min()) >= 0.0            # a maximum that started at 0 never falls below the gates' floor ...
    assert float(maxima.max()) > 1.0                    # ... and has moved


@pytest.mark.parametrize("E,top,count,keep", [(12, 3, 4, 2), (8, 8, 8, 8), (6, 1, 1, 1), (9, 2, 3, 1), (10, 4, 5, 3), (4, 2, 4, 2)])
def test_choice_of_experts(E, top, count, keep):
    """Sigmoid scores; a group counts by its two best (by its one expert where it has one); equal scores go to the
    lower index; the weights are the chosen scores over their sum, times the scale."""
    g = torch.Generator().manual_seed(E * 10 + top)
    z = torch.randn(40, E, generator=g, dtype=torch.float64) * 2
    z[3] = 0.0                                            # all equal
    z[4, 1::2] = z[4, 0::2][:len(z[4, 1::2])]             # pairs of equals
    idx, w = ops64().moe_route(z, None, top, count, keep, 1e-20, scoring="sigmoid", group_top=2, scale=1.7)
    for t in range(z.shape[0]):
        s = torch.sigmoid(z[t])
        chosen = plain.choose_experts(s, top, count, keep)
        assert idx[t].tolist() == chosen, t
        assert torch.allclose(w[t], s[chosen] / s[chosen].sum() * 1.7, atol=1e-14)


def test_the_two_maps_are_subtracted_and_normed():
    g = torch.Generator().manual_seed(7)
    N, H, G, P, Dv = 5, 6, 2, 16, 12
    o = torch.randn(N, 2 * H * P, generator=g, dtype=torch.float64)
    got = ops64().diff_combine(o, H, G, P, Dv, 0.37, 1e-5, 0.6)
    maps = o.view(N, G, 2, H // G, P)
    for h in range(H):
        y = maps[:, h // 3, 0, h % 3, :Dv] - 0.37 * maps[:, h // 3, 1, h % 3, :Dv]
        assert torch.allclose(got[:, h * Dv:(h + 1) * Dv], plain.rms(y, 1e-5) * 0.6, atol=1e-13)


# ---- edges --------------------------------------------------------------------------------------------
def _sharp(tmp_path, size=6, keep=3, scale=2.5, reader=None):
    layers = [differential(2, 1, 16, 8, size=size, keep=keep, rotation=rot(8, 1000.0, RAMP), diff=0.3, scale=scale)]
    if reader is not None:
        layers.append(differential(2, 1, 16, 8, size=reader[0], keep=reader[1], rotation=rot(8, 1000.0, RAMP), diff=0.6, scale=scale,
                                   kv_from=0))
    cfg = model(48, 50, layers, [moe(4, 2, 32, shared=24)] + [None] * (len(layers) - 1), embedding=2.0)
    return cfg, write_model(tmp_path / "sharp", cfg, seed=21)


def test_edges_of_the_window_and_of_the_kept_tokens_show(tmp_path):
    """A sharp softmax: the key just inside the window, or the last kept one, often carries the weight, so a window
    or a count of kept tokens that is one off moves the logits by far more than the tolerance. The plain model with
    the constants changed is the proof that the test can see each; the framework matches the unchanged one under
    every cut, in prompts and in decoding, in pages of 4 and of 16."""
    size, keep = 6, 3
    cfg, folder = _sharp(tmp_path, size, keep)
    prompts = random_prompts([60], cfg["vocab"], seed=22)
    want = oracle(folder, prompts)
    for cut in ("whole", "tail", "portions"):
        for bs in (4, 16):
            check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=bs, max_len=64, what=f"edges {cut}")
    pcfg, w = read_folder(folder)
    mask = pcfg["layers"][0]["mixer"]["mask"]
    for key, other in (("size", size - 1), ("size", size + 1), ("keep_first", keep - 1), ("keep_first", keep + 1)):
        was, mask[key] = mask[key], other
        off = plain.forward(pcfg, w, prompts[0]).float()
        mask[key] = was
        with pytest.raises(AssertionError):
            compare(off[size + keep:], want[0][size + keep:], 50 * TOL)
        compare(off[:size - 1], want[0][:size - 1], TOL)           # the first tokens see everything either way


@pytest.mark.parametrize("reader", [(3, 5), (11, 0), (6, 3), (1, 1)])
def test_a_layer_on_another_layers_cache_keeps_its_own_mask(tmp_path, reader):
    """The second layer has queries, mask and constants of its own and the first layer's keys and values: behind a
    narrower window with more kept tokens, a wider one with none, the same, and a window of one token. A pool of few
    pages of 4: what lies behind both windows comes back while the kept first tokens stay. The plain model with the
    reader's mask one off is outside the tolerance."""
    cfg, folder = _sharp(tmp_path, 6, 3, reader=reader)
    prompts = random_prompts([70], cfg["vocab"], seed=23)
    want = oracle(folder, prompts)
    for cut in ("tail", "portions"):
        check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=4, max_len=80, num_blocks=16,
                    what=f"reader {reader} {cut}")
    pcfg, w = read_folder(folder)
    mask = pcfg["layers"][1]["mixer"]["mask"]
    mask["size"] += 1
    with pytest.raises(AssertionError):
        compare(plain.forward(pcfg, w, prompts[0]).float()[12:], want[0][12:], 50 * TOL)


def test_the_first_tokens_of_a_memory(tmp_path):
    """Input gates that start shut (a bias of -6) or wide open (+6) under a maximum that starts at 0, and a large eps
    in the head norm, so that the size of a head's result before the norm matters: the first tokens of whole
    prompts, of prompts of one and two tokens, and of portions match the plain model. (Where the maximum starts
    cancels between the state and the denominator's floor but for the small constant in the denominator.)"""
    for n, bias in enumerate((-6.0, 6.0)):
        cfg = model(40, 50, [memory(2, 8, 12, 10.0)], [None], embedding=2.0, eps=1e-2)
        w = random_weights(cfg, 33)
        w["l0.mix.i.b"] = torch.full((2,), bias)
        folder = write_model(tmp_path / f"m{n}", cfg, 33, w)
        prompts = random_prompts([24, 1, 2], cfg["vocab"], seed=34)
        want = oracle(folder, prompts)
        for cut in ("whole", "tail", "portions"):
            check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, max_len=64, what=f"first tokens {cut}")
        pcfg, pw = read_folder(folder)
        other = plain.forward(pcfg, pw, prompts[0], first_max=-1e30).float()
        compare(other, want[0], 1e-3)


# ---- every mixer alone and mixtures, cut in every way -----------------------------------------------
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, name, cut):
    cfg = MODELS[name]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    pool = {}
    if cut == "mixed":
        # a pool that cannot hold all requests at once: pages come back and are used again
        pool = dict(num_blocks=4 * (-(-72 // BLOCK[name])))
    check_trace(folders[name], ops32(), prompts, CUTS[cut](prompts), TOL, block_size=BLOCK[name], max_len=128,
                what=f"{name} {cut}", **pool)


def test_a_batch_equals_each_request_alone(folders):
    cfg = MODELS["A"]
    prompts = random_prompts([37, 2, 19, 64], cfg["vocab"], seed=9)
    runner = make_runner(folders["A"], ops32(), max_len=128)
    alone = []
    for p in prompts:
        row = runner.cache.open_row()
        alone.append(runner.step([StepEntry(row, p, list(range(len(p))))]))
        runner.cache.close_row(row)
    rows = [runner.cache.open_row() for _ in prompts]
    together = runner.step([StepEntry(r, p, list(range(len(p)))) for r, p in zip(rows, prompts)])
    compare(together, torch.cat(alone), 1e-5, "batch against alone")


def test_rows_and_pages_used_again_start_clean(folders):
    """A state row (matrix, sum of keys, running maximum) and pages that another request left are taken by the next:
    its logits are those of a fresh run."""
    cfg = MODELS["A"]
    a, b = random_prompts([50, 33], cfg["vocab"], seed=11)
    runner = make_runner(folders["A"], ops32(), max_rows=1, max_len=64, block_size=4, num_blocks=16)
    want = oracle(folders["A"], [b])[0]
    for first in (a, b, a):
        row = runner.cache.open_row()
        runner.step([StepEntry(row, first, [])])
        runner.cache.close_row(row)
    row = runner.cache.open_row()
    assert row == 0
    got = torch.cat([runner.step([StepEntry(row, b[:20], list(range(20)))]), runner.step([StepEntry(row, b[20:], list(range(13)))])])
    compare(got, want, TOL, "a row used again")


def test_pages_behind_the_window_come_back_but_the_first_stay(folders):
    """120 tokens in pages of 4 would be 30 pages per layer; the windowed slot (which two layers read, behind 20 tokens
    and 2 kept ones at most) gives pages back, so a pool of 40 serves it beside the unmasked layer's 30."""
    cfg = MODELS["A"]
    prompts = random_prompts([120], cfg["vocab"], seed=24)
    runner = make_runner(folders["A"], ops32(), max_rows=1, max_len=128, block_size=4, num_blocks=40)
    want = oracle(folders["A"], prompts)[0]
    row = runner.cache.open_row()
    got, t = [], 0
    for n in [33, 2, 17, 1, 1, 30, 5, 31]:
        got.append(runner.step([StepEntry(row, prompts[0][t:t + n], list(range(n)))]))
        t += n
        runner.cache.check()
    assert t == 120
    compare(torch.cat(got), want, TOL, "a small pool")
    windowed = [g for g in runner.cache.groups if g.need.window is not None]
    assert len(windowed) == 1 and windowed[0].host_table[row, 0] != 0 and windowed[0].first_live[row] > 1
    assert windowed[0].held_count(row) <= 15             # (a portion of 31 tokens behind a window of 20, and the first page)
    runner.cache.close_row(row)
    runner.cache.check()


def test_a_token_far_back_reaches_through_the_memory(tmp_path):
    """Forget gates that hardly forget and no attention: what the first token was still shows 150 tokens later, in
    the plain model by far more than the tolerance, and the framework carries it through portions and single tokens."""
    cfg = model(48, 50, [memory(2, 24, 16, 12.0), memory(3, 8, 20, 12.0)], [moe(4, 2, 32), None], embedding=2.0)
    w = random_weights(cfg, 31)
    for name in w:
        if name.endswith("f.b"):
            w[name] = torch.full_like(w[name], 9.0)
        if name.endswith("mix.f"):
            w[name] = w[name] * 0.1
        if name.endswith("i.b"):
            w[name] = torch.tensor([3.0] + [-3.0] * (w[name].numel() - 1))
    folder = write_model(tmp_path / "m", cfg, 31, w)
    prompt = random_prompts([160], cfg["vocab"], seed=32)[0]
    other = [(prompt[0] + 7) % cfg["vocab"]] + prompt[1:]
    want, moved = oracle(folder, [prompt, other])
    with pytest.raises(AssertionError):
        compare(moved[150:], want[150:], 50 * TOL)
    for cut in ("portions", "tail"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=[want], max_len=192, what=f"far {cut}")


def test_a_far_key_among_hundreds(tmp_path):
    """Causal attention over 300 keys whose values are the keys: the key matrix is the query matrix behind a map that
    sends the input of the token at position 7 to that of the token at position 290, without rotation, so that key
    is what position 290 looks at, among hundreds, across page borders, in a prompt and decoded. Changing the token
    at 7 moves the logits at 290 by far more than the tolerance."""
    cfg = model(32, 40, [keyed(1, 1, 16, None, scale=3.0, softcap=100.0)], [None], embedding=1.0)
    w = random_weights(cfg, 41)
    prompt = [t % 38 for t in random_prompts([300], cfg["vocab"], seed=42)[0]]
    prompt[7], prompt[290] = 38, 39                        # two tokens that appear nowhere else
    e = w["embed"][[38, 39]].double()
    h = plain.rms(e, 1e-5) * w["l0.norm1"].double()
    turn = torch.eye(32, dtype=torch.float64) + torch.outer(h[1] - h[0], h[0]) / h[0].dot(h[0])
    w["l0.mix.k"] = (w["l0.mix.q"].double() @ turn).float()
    folder = write_model(tmp_path / "m", cfg, 41, w)
    want = oracle(folder, [prompt])
    moved = oracle(folder, [[1 if i == 7 else t for i, t in enumerate(prompt)]])
    with pytest.raises(AssertionError):
        compare(moved[0][290:291], want[0][290:291], 50 * TOL)
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=want, block_size=16, max_len=320, what=f"far key {cut}")


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    cfg = drawn_model(seed)
    folder = write_model(tmp_path / "m", cfg, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], cfg["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    # (such models can be touchy in float32: a sharp softmax, a width of 24; a fault is larger by far)
    check_trace(folder, ops32(), prompts, CUTS[["mixed", "portions", "tail"][seed % 3]](prompts), 5 * TOL, block_size=block,
                max_len=64, what=f"drawn {seed}")


def test_long_decoding(folders):
    """225 tokens one by one: the windows pass over decoded tokens, pages come back, the memory runs on."""
    cfg = MODELS["B"]
    prompts = random_prompts([230], cfg["vocab"], seed=25)
    steps = [([("r0", prompts[0][:5], list(range(5)))], [])]
    steps += [([("r0", [t], [0])], []) for t in prompts[0][5:]]
    steps[-1] = (steps[-1][0], ["r0"])
    check_trace(folders["B"], ops32(), prompts, steps, TOL, max_len=256, what="225 decoded tokens")


def test_greedy_generation_through_the_engine(folders):
    """The framework's own entry point and scheduler over this model: more requests than rows, prompts cut
    into portions, rows used again; the tokens are the plain model's greedy ones."""
    from socrates_amd.engine import Engine
    cfg, w = read_folder(folders["A"])
    prompts = random_prompts([12, 3, 29, 7, 18], cfg["vocab"], seed=26)
    want = [plain.greedy(cfg, w, p, 6) for p in prompts]
    runner = make_runner(folders["A"], ops64(), max_rows=3, max_len=64, block_size=4)
    engine = Engine(runner, device="cpu", dtype=torch.float64, compile=False, max_batch=3, max_len=64, max_new_tokens=6,
                    block_size=4, chunk=8)
    assert engine.generate(prompts, max_new_tokens=6) == want


def test_tokens_do_not_depend_on_the_pool(folders):
    """Pools so small that requests wait and have their portions shortened, or are preempted and computed again (their
    states cleared): float64 greedy tokens are those of a roomy pool and of the plain model."""
    from socrates_amd.engine import Engine
    cfg, w = read_folder(folders["B"])
    prompts = random_prompts([5, 17, 33, 9, 24, 40, 1, 12], cfg["vocab"], seed=27)
    want = [plain.greedy(cfg, w, p, 8) for p in prompts]

    def engine_with(num_blocks, chunk):
        runner = make_runner(folders["B"], ops64(), max_rows=4, max_len=64, block_size=4, num_blocks=num_blocks)
        return Engine(runner, device="cpu", dtype=torch.float64, compile=False, max_batch=4, max_len=64, max_new_tokens=8,
                      block_size=4, chunk=chunk)
    for num_blocks, chunk in ((64, 2048), (14, 7), (12, 5)):
        engine = engine_with(num_blocks, chunk)
        assert engine.generate(prompts, max_new_tokens=8) == want, (num_blocks, chunk)
        engine.cache.check()
        assert not engine.cache.open_rows and all(g.allocator.n_free == g.allocator.num_blocks for g in engine.cache.groups)
