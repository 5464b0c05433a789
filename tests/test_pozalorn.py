"""Pozalorn through the framework's step function, cache manager and scheduler, on the CPU with the
stand-in kernels, against the plain implementation in ``plain_pozalorn``: every mechanism alone and in
mixtures; whole prompts, token-by-token decoding, portions down to two tokens, mixed batches in a pool so
small that pages and state rows are used again; the edges of the windows and of the pooled blocks; the
sink of the softmax; far tokens through a state and through a block's mean; the configuration and the
weights' names."""

import json
import math

import pytest
import torch

import plain_pozalorn as plain
from helpers import make_runner, random_prompts
from pozalorn_models import (BLOCK, CUTS, MODELS, STRETCH, attention, check_trace, compare, dense, drawn_model, gla, lightning, model,
                             oracle, parallel, random_weights, read_folder, rot, tensor_shapes, window, write_model)
from socrates_amd.config import ConfigError, load_config
from socrates_amd.config.pozalorn import PozalornConfig
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
    base = tmp_path_factory.mktemp("pozalorn")
    return {name: write_model(base / name, made, seed=i + 1) for i, (name, made) in enumerate(MODELS.items())}


# ---- configuration, plan, names ---------------------------------------------------------------------
def test_plan_follows_the_configuration(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, PozalornConfig) and cfg.to_dict() == MODELS["A"][0]
    plan = cfg.plan()
    needs = cache_needs(plan)
    assert isinstance(needs[0], RowState) and needs[0].shape == (2 * 16 * 32,)
    # keys of 32 beside values of 16 share pools of 32, with the means of blocks of 4
    assert needs[1] == PagedKV(1, 32, 9, 0, 4)
    # two mixers side by side: the window's pages (keys of 16 beside values of 24 take 32) and the state
    assert needs[2][0] == PagedKV(2, 32, 5, 0, 0) and needs[2][1].shape == (3 * 8 * 8,)
    assert needs[3] == PagedKV(2, 48, 12, 0, 16)
    assert plan.layers[1].ffn is None and "l1.norm2" in plan.ignorable
    names = expected_tensors(plan)
    want = tensor_shapes(MODELS["A"])
    assert set(names) == set(want)
    assert all(names[n].fits(want[n]) for n in want), [n for n in want if not names[n].fits(want[n])]


def test_configuration_errors():
    good = MODELS["A"][0]

    def broken(change):
        bad = json.loads(json.dumps(good))
        change(bad)
        return bad
    with pytest.raises(ConfigError, match="unknown type"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][0].update(type="conv")))
    with pytest.raises(ConfigError, match="decay"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][2]["mixer"]["right"].update(decay=[0.5])))
    with pytest.raises(ConfigError, match="rot.dims"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34)))
    with pytest.raises(ConfigError, match="kv heads"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=2)))
    with pytest.raises(ConfigError, match="lacks"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][0]["mixer"].pop("tau")))
    with pytest.raises(ConfigError, match="lacks"):
        PozalornConfig.from_dict(broken(lambda c: c.pop("norm")))
    with pytest.raises(ConfigError, match="feed-forward"):
        PozalornConfig.from_dict(broken(lambda c: c["layers"][0]["mlp"].update(kind="moe")))


# ---- each mechanism of the stand-in kernel set against the plain function ---------------------------------
@pytest.mark.parametrize("dims,base,stretch", [(16, 300000.0, (6.0, 1.0, 4.0, 32)), (48, 40000.0, (3.0, 1.0, 8.0, 4096)), (8, 100.0, None),
                                               (24, 10000.0, (2.0, 2.0, 16.0, 64)), (2, 7.0, (3.0, 1.0, 2.0, 4))])
def test_stretched_frequencies(dims, base, stretch):
    """Short wavelengths stay, long ones are divided, and those between slide from the one to the other."""
    scaling = None if stretch is None else dict(zip(("factor", "low", "high", "original"), stretch))
    want = plain.frequencies(dims, base, scaling)
    got = torch.tensor(PairRopeSpec(dims=dims, base=base, stretch=stretch).frequencies(), dtype=torch.float64)
    assert torch.allclose(got, want, rtol=1e-13, atol=0)
    if stretch is not None and dims >= 16:
        plainest = plain.frequencies(dims, base)
        ratio = want / plainest
        assert float(ratio.max()) <= 1.0 and float(ratio.min()) == pytest.approx(1.0 / stretch[0])
        assert float(ratio[0]) == 1.0 or 2 * math.pi >= stretch[3] / stretch[2]     # the shortest wave stays where it is short enough
        assert ((ratio < 1.0) & (ratio > 1.0 / stretch[0])).any()                   # somewhere between the two


def _ctx(lengths, rows, starts):
    from types import SimpleNamespace
    q = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lengths)]).to(torch.int32)
    trow = torch.cat([torch.full((n,), r) for r, n in zip(rows, lengths)]).to(torch.int32)
    return SimpleNamespace(n_seqs=len(lengths), n_tokens=int(q[-1]), seq_qstart=q, seq_rows=torch.tensor(rows, dtype=torch.int32),
                           positions=pos, token_rows=trow, max_q_len=max(lengths),
                           seq_ctx=torch.tensor([s + n for s, n in zip(starts, lengths)], dtype=torch.int32),
                           max_ctx_len=max(s + n for s, n in zip(starts, lengths)))


@pytest.mark.parametrize("channel", [False, True])
def test_linear_attention_in_portions_equals_the_plain_recurrence(channel):
    """One sequence of 23 tokens in portions of 9, 1, 2 and 11 beside another sequence, from the state that each
    portion left: the plain function over the whole sequence, for a decay per head and for one per channel and token."""
    g = torch.Generator().manual_seed(4)
    H, D, Dv, T = 3, 5, 7, 23
    x = torch.randn(T, 2 * H * D + H * Dv, generator=g, dtype=torch.float64)
    other = torch.randn(T, 2 * H * D + H * Dv, generator=g, dtype=torch.float64)
    z = torch.randn(T, H * D, generator=g, dtype=torch.float64)
    zb = torch.randn(H * D, generator=g, dtype=torch.float64)
    decays = torch.tensor([0.5, 0.9, 1.0], dtype=torch.float64)
    q, k, v = x[:, :H * D].view(T, H, D), x[:, H * D:2 * H * D].view(T, H, D), x[:, 2 * H * D:].view(T, H, Dv)
    if channel:
        want = plain.linear_attention(q * 0.3, k, v, torch.sigmoid(z + zb).pow(1 / 4.0).view(T, H, D))
    else:
        want = plain.linear_attention(plain.silu(q) * 0.3, plain.silu(k), plain.silu(v), decays[None, :, None].expand(T, H, D))
    state = torch.zeros(4, 2 + H * D * Dv, dtype=torch.float64)
    got, t = [], 0
    for n in (9, 1, 2, 11):
        ctx = _ctx([n, n], [2, 0], [t, t])
        xs = torch.cat([x[t:t + n], other[t:t + n]])
        zs = torch.cat([z[t:t + n], z[t:t + n]])
        out = ops64().linear_attention(xs, (0, H * D, 2 * H * D), H, D, Dv, 0.3, not channel, None if channel else decays,
                                       zs if channel else None, zb if channel else None, 4.0, state, 2, ctx)
        got.append(out[:n])
        t += n
    assert torch.allclose(torch.cat(got).view(T, H, Dv), want, atol=1e-12)
    assert float(state[:, :2].abs().max()) == 0.0 and float(state[1].abs().max()) == 0.0


def test_gelu_gate_and_sums():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(9, 14, generator=g, dtype=torch.float64) * 3
    want = plain.gelu_tanh(x[:, :5]) * x[:, 5:10]
    assert torch.allclose(ops64().glu_gelu(x, 5), want, atol=1e-13)
    assert torch.allclose(plain.gelu_tanh(torch.tensor([1.0], dtype=torch.float64)), torch.tensor([0.8411919906], dtype=torch.float64), atol=1e-9)
    a, b, bias = x[:, :4], x[:, 4:8], x[0, 8:12]
    assert torch.allclose(ops64().scaled_sum(a, 0.8, b, 1.1, bias), 0.8 * (a + bias) + 1.1 * b, atol=1e-13)
    # results by depth: after layer i the stream is a weighted sum of the embedding output and the results so far
    kept = ops64().depth_begin(a.clone(), 3)
    r = b.clone()
    ops64().depth_average(r, kept, 1, torch.tensor([0.3, -0.7], dtype=torch.float64), cast=False)
    assert torch.allclose(r, 0.3 * a - 0.7 * b, atol=1e-13)
    later = x[:, 10:14].clone()
    ops64().depth_average(later, kept, 2, torch.tensor([0.1, 0.2, 0.5], dtype=torch.float64), cast=False)
    assert torch.allclose(later, 0.1 * a + 0.2 * b + 0.5 * x[:, 10:14], atol=1e-13)      # the results themselves are kept, not the sums


def test_the_sink_counts_once_and_has_no_value():
    s = torch.tensor([[0.3, -1.0, 2.0, 0.5]], dtype=torch.float64)
    seen = torch.tensor([[True, True, False, True]])
    p = plain.softmax_over(s, seen, torch.tensor(0.7, dtype=torch.float64))
    e = torch.exp(torch.tensor([0.3, -1.0, 0.5], dtype=torch.float64))
    assert torch.allclose(p[0, [0, 1, 3]], e / (e.sum() + math.exp(0.7)), atol=1e-14) and float(p[0, 2]) == 0.0


# ---- edges --------------------------------------------------------------------------------------------
def _sharp_pooled(tmp_path, size=6, pool=4, scale=2.5):
    made = model(48, 50, [attention(2, 1, 16, 8, size=size, pool=pool, rotation=rot(8, 1000.0, STRETCH), scale=scale)], [dense(64)])
    folder = write_model(tmp_path / "pooled", made, seed=21)
    return made, folder


def test_edges_of_the_window_and_of_the_pooled_blocks_show(tmp_path):
    """A sharp softmax: the key just inside the window, or the block that has just come into sight, often carries
    the weight, so a window or a block one off moves the logits by far more than the tolerance. The plain model
    with the constants changed is the proof that the test can see each; the framework matches the unchanged one
    under every cut, in prompts and in decoding, in pages of 4 (a block of 4 is a page) and of 16."""
    size, pool = 6, 4
    made, folder = _sharp_pooled(tmp_path, size, pool)
    prompts = random_prompts([60], made[0]["vocab"], seed=22)
    want = oracle(folder, prompts)
    for cut in ("whole", "tail", "portions"):
        for bs in (4, 16):
            check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=bs, max_len=64, what=f"edges {cut}")
    pcfg, w = read_folder(folder)
    mask = pcfg["layers"][0]["mixer"]["mask"]
    for key, other in (("size", size - 1), ("size", size + 1), ("pool", pool - 1), ("pool", pool + 1)):
        was, mask[key] = mask[key], other
        off = plain.forward(pcfg, w, prompts[0]).float()
        mask[key] = was
        with pytest.raises(AssertionError):
            compare(off[size + pool:], want[0][size + pool:], 50 * TOL)
        compare(off[:size - 1], want[0][:size - 1], TOL)           # the first tokens see everything either way
    # a block comes into sight exactly when its last token has left the window
    seen_blocks = [max(0, (i - size + 1) // pool) for i in range(20)]
    assert seen_blocks[size + pool - 2] == 0 and seen_blocks[size + pool - 1] == 1


@pytest.mark.parametrize("size,pool", [(5, 7), (3, 1), (16, 16), (1, 2), (10, 3)])
def test_blocks_and_windows_of_every_relation(tmp_path, size, pool):
    """Blocks longer than the window, of one token, equal to the window and to a page, a window of one token, a
    block that divides neither window nor page; pages of 4, so blocks span pages and pages span blocks."""
    made = model(40, 45, [attention(4, 2, 8, 12, size=size, pool=pool, rotation=rot(4, 300.0), scale=0.9)], [None])
    folder = write_model(tmp_path / "m", made, seed=size * 20 + pool)
    prompts = random_prompts([50, 2, 33], made[0]["vocab"], seed=23)
    want = oracle(folder, prompts)
    for cut in ("tail", "portions", "mixed"):
        check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=4, max_len=64, what=f"{size}/{pool} {cut}")


def test_the_sink_and_the_window_of_the_left_side_show(tmp_path):
    size = 5
    made = model(48, 50, [parallel(window(4, 2, 12, 8, size, rot(6, 1000.0, STRETCH), scale=1.5), lightning(2, 8, 8, (0.9, 0.8)), 1.2, 0.5)],
                 [dense(64)])
    w = random_weights(made, 24)
    w["l0.mix.left.sink"] = torch.tensor([2.0, -1.0, 3.0, 0.5])
    folder = write_model(tmp_path / "m", made, 24, w)
    prompts = random_prompts([48], made[0]["vocab"], seed=25)
    want = oracle(folder, prompts)
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), prompts, CUTS[cut](prompts), TOL, want=want, block_size=4, max_len=64, what=f"sink {cut}")
    pcfg, pw = read_folder(folder)
    mask = pcfg["layers"][0]["mixer"]["left"]["mask"]
    for other in (size - 1, size + 1):
        mask["size"] = other
        with pytest.raises(AssertionError):
            compare(plain.forward(pcfg, pw, prompts[0]).float()[size:], want[0][size:], 50 * TOL)
    mask["size"] = size
    pw["l0.mix.left.sink"] = torch.full((4,), -1e9, dtype=torch.float64)       # no sink: also the very first token shows it
    without = plain.forward(pcfg, pw, prompts[0]).float()
    with pytest.raises(AssertionError):
        compare(without[:1], want[0][:1], 50 * TOL)
    with pytest.raises(AssertionError):
        compare(without[size:], want[0][size:], 50 * TOL)


# ---- every mixer alone and mixtures, cut in every way -----------------------------------------------
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, name, cut):
    cfg = MODELS[name][0]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    pool = {}
    if cut == "mixed":
        # a pool that cannot hold all requests at once: pages come back and are used again
        pool = dict(num_blocks=4 * (-(-72 // BLOCK[name])))
    check_trace(folders[name], ops32(), prompts, CUTS[cut](prompts), TOL, block_size=BLOCK[name], max_len=128,
                what=f"{name} {cut}", **pool)


def test_a_batch_equals_each_request_alone(folders):
    cfg = MODELS["A"][0]
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
    """A state row, pages and pages of means that another request left are taken by the next: its logits are
    those of a fresh run."""
    cfg = MODELS["A"][0]
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


def test_pages_behind_the_window_come_back_but_the_means_stay(folders):
    """120 tokens in pages of 4 would be 30 pages per layer; behind windows of at most 12 tokens (and blocks of at
    most 16 that wait for their last token) a pool of 18 serves portions of up to 33 tokens. The means of all
    blocks are still the row's at the end, the tokens' pages behind the window are not."""
    cfg = MODELS["A"][0]
    prompts = random_prompts([120], cfg["vocab"], seed=24)
    runner = make_runner(folders["A"], ops32(), max_rows=1, max_len=128, block_size=4, num_blocks=18)
    want = oracle(folders["A"], prompts)[0]
    row = runner.cache.open_row()
    got, t = [], 0
    for n in [33, 2, 17, 1, 1, 30, 5, 31]:
        got.append(runner.step([StepEntry(row, prompts[0][t:t + n], list(range(n)))]))
        t += n
        runner.cache.check()
    assert t == 120
    compare(torch.cat(got), want, TOL, "a small pool")
    tokens = [g for g in runner.cache.groups if not g.means]
    means = [g for g in runner.cache.groups if g.means]
    assert len(means) == 2 and all(g.host_table[row, 0] != 0 for g in means)
    assert sorted(g.covered[row] for g in means) == sorted(-(-(120 // g.per) // 4) for g in means)
    assert tokens and all(g.host_table[row, 0] == 0 and g.first_live[row] > 0 for g in tokens)
    runner.cache.close_row(row)
    runner.cache.check()
    assert all(g.allocator.n_free == g.allocator.num_blocks - 1 or g.allocator.n_free == g.allocator.num_blocks for g in runner.cache.groups)


def test_a_token_far_back_reaches_through_the_states(tmp_path):
    """Slow decays and no softmax attention to speak of (a window of one token): what the first token was still
    shows 150 tokens later, in the plain model by far more than the tolerance, and the framework carries it
    through portions and single tokens, in the state of gated linear attention and in that of lightning attention."""
    for n, layers in enumerate(([gla(2, 24, 16, 64.0, rank=4), gla(3, 8, 20, 32.0, rank=2)],
                                [parallel(window(1, 1, 4, 4, 1, rot(2)), lightning(2, 24, 16, (0.995, 1.0)), 0.1, 1.0)] * 2)):
        made = model(48, 50, layers, [dense(64), None])
        w = random_weights(made, 31 + n)
        for name in w:
            if name.endswith("a2.b"):
                w[name] = w[name] + 3.0          # decays near one
        folder = write_model(tmp_path / f"m{n}", made, 31, w)
        prompt = random_prompts([160], made[0]["vocab"], seed=32)[0]
        other = [(prompt[0] + 7) % made[0]["vocab"]] + prompt[1:]
        want, moved = oracle(folder, [prompt, other])
        with pytest.raises(AssertionError):
            compare(moved[150:], want[150:], 50 * TOL)
        for cut in ("portions", "tail"):
            check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=[want], max_len=192, what=f"far {cut}")


def test_a_far_block_among_many(tmp_path):
    """A window of 8 tokens behind 200, blocks of 4: the key matrix is the query matrix behind a map that sends the
    input of the token that fills block 1 (positions 4 to 7) to that of the token at position 190, without
    rotation of q and k, so that block's mean is what position 190 looks at, among 45 blocks, across page borders,
    in a prompt and decoded. Changing the tokens of that block moves the logits at 190 by far more than the
    tolerance; changing them at 189, where another query looks, does not."""
    made = model(32, 40, [attention(1, 1, 16, 16, size=8, pool=4, rotation=rot(0, 10000.0), scale=1.5)], [None])
    w = random_weights(made, 41)
    prompt = [t % 38 for t in random_prompts([200], made[0]["vocab"], seed=42)[0]]
    prompt[4:8] = [38] * 4
    prompt[190] = 39                                       # two tokens that appear nowhere else
    h = w["embed"][[38, 39]].double()
    turn = torch.eye(32, dtype=torch.float64) + torch.outer(h[1] - h[0], h[0]) / h[0].dot(h[0])
    w["l0.mix.k"] = (w["l0.mix.q"].double() @ turn).float()
    w["l0.mix.k.b"], w["l0.mix.k.norm"] = w["l0.mix.q.b"].clone(), w["l0.mix.q.norm"].clone()
    folder = write_model(tmp_path / "m", made, 41, w)
    want = oracle(folder, [prompt])
    moved = oracle(folder, [[1 if 4 <= i < 8 else t for i, t in enumerate(prompt)]])
    with pytest.raises(AssertionError):
        compare(moved[0][190:191], want[0][190:191], 50 * TOL)
    compare(moved[0][20:190], want[0][20:190], 0.25)       # elsewhere that block is one among many
    for cut in ("whole", "tail", "portions"):
        check_trace(folder, ops32(), [prompt], CUTS[cut]([prompt]), TOL, want=want, block_size=16, max_len=256, what=f"far block {cut}")


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    made = drawn_model(seed)
    folder = write_model(tmp_path / "m", made, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], made[0]["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    # (such models can be touchy in float32: a sharp softmax, a width of 24, a decay of one; a fault is larger by far)
    check_trace(folder, ops32(), prompts, CUTS[["mixed", "portions", "tail"][seed % 3]](prompts), 5 * TOL, block_size=block,
                max_len=64, what=f"drawn {seed}")


def test_long_decoding(folders):
    """225 tokens one by one: the windows pass over decoded tokens, blocks come into sight, pages come back, the
    states run on."""
    cfg = MODELS["B"][0]
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
    runner = make_runner(folders["A"], ops32(), max_rows=3, max_len=64, block_size=4)
    engine = Engine(runner, device="cpu", dtype=torch.float32, compile=False, max_batch=3, max_len=64, max_new_tokens=6,
                    block_size=4, chunk=8)
    assert engine.generate(prompts, max_new_tokens=6) == want


def test_tokens_do_not_depend_on_the_pool(folders):
    """Pools so small that requests wait and have their portions shortened, and two requests that fit at admission and
    outgrow the pool while decoding behind a window longer than they are: the younger is preempted and computed again
    (its states cleared, its means taken anew). float64 greedy tokens are those of a roomy pool and of the plain model."""
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
    engine = engine_with(7, 64)
    assert engine.generate([prompts[7], prompts[3]], max_new_tokens=8) == [want[7], want[3]]
    assert engine.scheduler.n_preemptions > 0
    engine.cache.check()
