"""Berelorn on the GPU: every new or extended HIP kernel against its stand-in from odd sizes and non-zero states,
then the kernels under the framework's step function, cache manager, scheduler and entry points, in float32 and
bfloat16, against the plain implementation in ``plain_berelorn``: the same small models and cuts as on the CPU,
captured decode steps, greedy generation through ``Engine`` and the trace runner as a user starts it."""

import json
import subprocess
import sys
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_berelorn as plain
from berelorn_models import (BLOCK, CUTS, MODELS, RAMP, check_trace, compare, differential, drawn_model, keyed, memory, model, moe,
                             oracle, read_folder, rot, row_errors, write_model)
from helpers import make_runner, random_prompts, replay, trace_mixed, trace_portions, trace_tail_decode
from torch_kernels import TorchKernels

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# in units of the logits' spread per position; bfloat16: (every row, nine rows in ten). A token whose choice of experts
# hangs on less than bfloat16 resolves may choose otherwise than the plain model, which moves that row.
TOL = {"float32": 3e-4, "bfloat16": (0.6, 0.06)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("berelorn_gpu")
    return {name: write_model(base / name, cfg, seed=i + 1) for i, (name, cfg) in enumerate(MODELS.items())}


@pytest.fixture(scope="module")
def kernel_sets():
    from socrates_amd.kernels import HipKernels
    return {name: HipKernels(dt, DEV) for name, dt in DTYPES.items()}


def _close(got, want, dtype, what, scale=1.0):
    tol = dict(atol=2e-5 * scale, rtol=2e-5) if dtype == "float32" else dict(atol=2e-2 * scale, rtol=2e-2)
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), msg=lambda m: f"{what} ({dtype}): {m}", **tol)


def _ctx(lengths, rows, starts, dev):
    """A step's context for kernels that walk sequences: tokens of several sequences one after the other."""
    q = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    pos = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, lengths)]).astype(np.int32)
    trow = np.concatenate([np.full(n, r) for r, n in zip(rows, lengths)]).astype(np.int32)
    t = lambda a: torch.as_tensor(np.asarray(a), dtype=torch.int32, device=dev)      # noqa: E731
    return SimpleNamespace(n_seqs=len(lengths), n_tokens=int(q[-1]), seq_qstart=t(q), seq_rows=t(rows), positions=t(pos),
                           token_rows=t(trow), max_q_len=int(max(lengths)), seq_ctx=t([s + n for s, n in zip(starts, lengths)]),
                           max_ctx_len=int(max(s + n for s, n in zip(starts, lengths))))


# ---- each kernel against its stand-in ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("H,D,Dv", [(3, 20, 28), (1, 48, 80), (4, 8, 8), (2, 64, 40), (2, 128, 64), (1, 200, 15), (6, 32, 63)])
@pytest.mark.parametrize("lengths", [[9, 1, 2, 15], [37, 1, 2, 170], [300, 1, 64, 65], [2300, 17, 1, 1024]])
def test_matrix_memory_kernels(kernel_sets, dtype, H, D, Dv, lengths):
    """The gates with their running maximum over several sequences of unequal length (more than a wave of tokens among
    them, and single tokens) from maxima that are not zero; the recurrence over prepared q, k and decays with the
    sum of keys as one more column, from a state that is not zero; denominators, head norms, gain and gate."""
    ops, dt = kernel_sets[dtype], DTYPES[dtype]
    ref = TorchKernels(dt, DEV)
    g = torch.Generator(device="cpu").manual_seed(H * D + Dv)
    if max(lengths) > 1000 and D * Dv > 2000:
        pytest.skip("the longest portions with the small states only (the stand-in walks token by token)")
    rows, starts = [2, 0, 3, 1], [5, 300, 0, 41]
    ctx = _ctx(lengths, rows, starts, DEV)
    N, ld = ctx.n_tokens, 7 + H * (2 * D + 2 * Dv)
    x = (torch.randn(N, ld, generator=g) * 0.7).to(dt).to(DEV)
    cols = (7 + H * Dv, 7 + H * Dv + H * D, 7 + H * Dv + 2 * H * D)
    gates = (torch.randn(N, 2 * H, generator=g) * 4).to(DEV)
    bias = torch.randn(2 * H, generator=g).to(DEV)
    n_state = H * D * (Dv + 1)
    state = torch.randn(5, 3 + n_state + H, generator=g).to(DEV)
    s1, s2 = state.clone(), state.clone()
    p1, m1 = ops.memory_gates(gates, bias, 7.0, x, cols, H, D, D ** -0.5, s1, 3 + n_state, ctx)
    p2, m2 = ref.memory_gates(gates, bias, 7.0, x, cols, H, D, D ** -0.5, s2, 3 + n_state, ctx)
    assert p1.dtype == torch.float32 and m1.dtype == torch.float32
    torch.testing.assert_close(p1.cpu(), p2.float().cpu(), atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(m1.cpu(), m2.float().cpu(), atol=2e-5, rtol=2e-5)
    got = ops.linear_attention(x, cols, H, D, Dv + 1, 1.0, False, None, None, None, 1.0, s1, 3, ctx, prepared=p2.float().contiguous(), ones=1)
    want = ref.linear_attention(x, cols, H, D, Dv + 1, 1.0, False, None, None, None, 1.0, s2, 3, ctx, prepared=p2, ones=1)
    torch.testing.assert_close(got.cpu(), want.float().cpu(), atol=3e-4, rtol=3e-4)
    torch.testing.assert_close(s1.cpu(), s2.cpu(), atol=3e-4, rtol=3e-4)
    assert torch.equal(s1[4], state[4]) and torch.equal(s1[:, :3], state[:, :3])       # rows and columns that are not the step's
    gain = (1 + 0.3 * torch.randn(H * Dv, generator=g)).to(DEV)
    raw = want.float().contiguous()
    _close(ops.memory_finish(raw, m2.float().contiguous(), x, gain, H, Dv, 1e-5, 1e-6),
           ref.memory_finish(raw, m2, x, gain, H, Dv, 1e-5, 1e-6), dtype, "denominators, norms and gate")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("H,G,P,Dv", [(6, 2, 16, 12), (4, 4, 64, 64), (3, 1, 48, 33), (8, 2, 256, 200), (1, 1, 16, 1)])
def test_the_two_maps_combined(kernel_sets, dtype, H, G, P, Dv):
    ops, dt = kernel_sets[dtype], DTYPES[dtype]
    g = torch.Generator(device="cpu").manual_seed(H + P)
    o = torch.randn(37, 2 * H * P, generator=g).to(dt).to(DEV)
    _close(ops.diff_combine(o, H, G, P, Dv, 0.37, 1e-5, 0.6), TorchKernels(dt, DEV).diff_combine(o, H, G, P, Dv, 0.37, 1e-5, 0.6),
           dtype, "a1 - lambda a2, normed")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("Hq,Hkv,D,Dv,rotary,tied", [(4, 2, 24, 12, 8, False), (3, 1, 16, 16, 16, True), (2, 2, 40, 40, 0, True),
                                                     (8, 8, 48, 32, 24, False), (1, 1, 200, 200, 100, True), (8, 2, 64, 64, 64, True)])
@pytest.mark.parametrize("norm", ["turned", None])
def test_prepare_kernel_with_a_norm_behind_the_rotation(kernel_sets, dtype, norm, Hq, Hkv, D, Dv, rotary, tied):
    """Cosines and sines with a magnitude, a norm per head behind the rotation without gains, values read from the
    keys' columns as projected, and queries alone with no cache slot."""
    from socrates_amd.cache.manager import PagedSlot
    from socrates_amd.config.specs import PairRopeSpec
    ops, dt = kernel_sets[dtype], DTYPES[dtype]
    ref = TorchKernels(dt, DEV)
    g = torch.Generator(device="cpu").manual_seed(D + Dv)
    P = (max(D, Dv) + 15) // 16 * 16
    ctx = _ctx([9, 1, 14], [1, 2, 0], [3, 17, 0], DEV)
    N, ld = ctx.n_tokens, 5 + Hq * D + Hkv * (D + Dv) + 3
    x = torch.randn(N, ld, generator=g).to(dt).to(DEV)
    cols = (5, 5 + Hq * D, 5 + Hq * D if tied else 5 + Hq * D + Hkv * D)
    bias = (0.5 * torch.randn(ld, generator=g)).to(DEV) if Hq != 3 else None
    inv_freq, magnitude = None, 1.0
    if rotary:
        spec = PairRopeSpec(dims=rotary, base=500.0, ramp=(4.0, 64, 8.0, 1.0))
        inv_freq, magnitude = torch.tensor(spec.frequencies(), dtype=torch.float64).float().to(DEV), spec.magnitude
    table = torch.zeros(4, 8, dtype=torch.int32, device=DEV)
    table[:3, :6] = torch.arange(1, 19, dtype=torch.int32, device=DEV).view(3, 6)
    outs = []
    for o in (ops, ref):
        slot = PagedSlot(torch.full((19, Hkv, 4, P), 7.0, dtype=dt, device=DEV), torch.full((19, Hkv, 4, P), 7.0, dtype=dt, device=DEV),
                         table, 4, None)
        q = o.window_prepare(x, cols, Hq, Hkv, D, Dv, P, bias, None, None, norm, 1e-5, inv_freq, rotary, None, ctx.positions,
                             ctx.token_rows, slot, magnitude=magnitude)
        alone = o.window_prepare(x, cols, Hq, 0, D, Dv, P, bias, None, None, norm, 1e-5, inv_freq, rotary, None, ctx.positions,
                                 ctx.token_rows, None, magnitude=magnitude)
        outs.append((q, slot.k, slot.v, alone))
    for a, b, what in zip(outs[0], outs[1], ("q", "keys", "values", "queries alone")):
        _close(a, b, dtype, what, scale=3.0)
    assert torch.equal(outs[0][0], outs[0][3])
    assert float(outs[0][1][0].float().abs().max()) == 7.0                  # the null page is nobody's


@pytest.mark.parametrize("P,G", [(64, 2), (128, 4), (48, 1), (32, 8)])
@pytest.mark.parametrize("row_tiles", [None, 1, 2, 32, 64])
@pytest.mark.parametrize("window,keep", [(None, 0), (90, 5)])
def test_a_soft_cap_in_the_attention_kernels_on_the_matrix_cores(kernel_sets, P, G, row_tiles, window, keep):
    """bfloat16 scores under a soft cap that bites (scores of several times the cap's size): long portions through every
    form of the kernel that shares its key tiles among four waves (one from position 0, one behind 300 cached tokens,
    also behind a window with kept first keys), single tokens behind long contexts through the per-wave kernel with
    its key splits, against the stand-in."""
    from socrates_amd.cache.manager import PagedSlot
    ops, dt = kernel_sets["bfloat16"], torch.bfloat16
    if row_tiles in (32, 64) and P % 32:
        pytest.skip("32-row products take head sizes in steps of 32")
    if row_tiles == 64 and keep:
        pytest.skip("no kept keys with the keys in two halves")
    ref = TorchKernels(dt, DEV)
    g = torch.Generator(device="cpu").manual_seed(P + G)
    Hkv, bs, pages = 2, 16, 48
    Hq = Hkv * G
    table = torch.arange(1, 1 + 5 * pages, dtype=torch.int32, device=DEV).view(5, pages)
    table = torch.cat([table, torch.zeros(1, pages, dtype=torch.int32, device=DEV)]).contiguous()
    slot = PagedSlot((torch.randn(1 + 5 * pages, Hkv, bs, P, generator=g) * 0.8).to(dt).to(DEV),
                     torch.randn(1 + 5 * pages, Hkv, bs, P, generator=g).to(dt).to(DEV), table, bs, window)
    terms = {"softcap": 3.0}
    if keep:
        terms["keep_first"] = keep
    for lengths, rows, starts in (([700, 1, 230, 1, 17], [0, 1, 2, 3, 4], [0, 59, 300, 5, 140]),
                                  ([1, 1, 1, 1], [0, 1, 2, 4], [699, 0, 530, 17])):
        ctx = _ctx(lengths, rows, starts, DEV)
        q = torch.randn(ctx.n_tokens, Hq, P, generator=g).to(dt).to(DEV)
        want = ref.paged_attention(q, slot, ctx, 1.0, window, terms=terms)
        uncapped = ref.paged_attention(q, slot, ctx, 1.0, window, terms={k: v for k, v in terms.items() if k != "softcap"} or None)
        assert float((want.float() - uncapped.float()).abs().max()) > 0.2          # the cap matters here
        ops.attention_row_tiles = row_tiles if max(lengths) > 1 else None
        try:
            got = ops.paged_attention(q, slot, ctx, 1.0, window, terms=terms)
            kernel = ops.last_attention_kernel
        finally:
            ops.attention_row_tiles = None
        if max(lengths) > 1 and row_tiles:
            assert kernel == ("workgroup", row_tiles)
        elif not keep:
            assert kernel[0] == "wave"
        _close(got, want, "bfloat16", f"soft cap, window {window}, {keep} kept, row tiles {row_tiles} ({kernel})")


@pytest.mark.parametrize("E,top,count,keep,group_top", [(12, 3, 4, 2, 2), (8, 8, 8, 8, 2), (6, 1, 1, 1, 2), (9, 2, 3, 1, 3), (200, 6, 20, 7, 2),
                                                        (256, 8, 1, 1, 1), (10, 4, 5, 3, 1)])
def test_choice_of_experts_kernel(kernel_sets, E, top, count, keep, group_top):
    """Sigmoid scores from columns of a wider product, groups scored by the sum of their best, equal scores, the scale."""
    ops = kernel_sets["float32"]
    g = torch.Generator(device="cpu").manual_seed(E + top)
    wide = (torch.randn(70, E + 3, generator=g) * 2).to(DEV)
    wide[3] = 0.0
    wide[4, 1:E:2] = wide[4, 0:E:2][:len(wide[4, 1:E:2])]
    z = wide[:, :E]
    for scoring in ("sigmoid", "softmax"):
        idx, w = ops.moe_route(z, None, top, count, keep, 1e-20, scoring=scoring, group_top=group_top, scale=1.7)
        ridx, rw = TorchKernels(torch.float32, DEV).moe_route(z.contiguous(), None, top, count, keep, 1e-20, scoring=scoring,
                                                              group_top=group_top, scale=1.7)
        # (a choice may hang on the last bit of a score or of a group's sum: nearly all rows agree, and the rows of
        # equal scores, where the lower index wins, agree exactly)
        same = (idx == ridx).all(-1)
        assert same.float().mean() > 0.9 and bool(same[3]) and (bool(same[4]) or scoring == "softmax")
        torch.testing.assert_close(w[same], rw[same], atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("N,E,top,d,ff", [(7, 5, 2, 48, 24), (150, 6, 3, 64, 40), (700, 4, 1, 128, 64), (33, 9, 9, 40, 20)])
def test_silu_gated_experts_and_a_gated_shared_term(kernel_sets, dtype, N, E, top, d, ff):
    ops, dt = kernel_sets[dtype], DTYPES[dtype]
    ref = TorchKernels(dt, DEV)
    g = torch.Generator(device="cpu").manual_seed(N + E)
    x = torch.randn(N, d, generator=g).to(dt).to(DEV)
    w1 = (torch.randn(E, 2 * ff, d, generator=g) / d ** 0.5).to(dt).to(DEV)
    w2 = (torch.randn(E, d, ff, generator=g) / ff ** 0.5).to(dt).to(DEV)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(N)]).to(torch.int32).to(DEV)
    weight = torch.rand(N, top, generator=g).to(DEV)
    extra = torch.randn(N, d, generator=g).to(dt).to(DEV)
    wide = torch.randn(N, 3, generator=g).to(DEV)
    got = ops.moe_experts(x, idx, weight, w1, w2, 3.0e38, 1.0, extra, shift=0.0, extra_gate=wide[:, 2])
    want = ref.moe_experts(x, idx, weight, w1, w2, 3.0e38, 1.0, extra, shift=0.0, extra_gate=wide[:, 2])
    assert got.dtype == torch.float32
    _close(got, want, dtype, "experts", scale=2.0)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("d", [40, 192, 1000, 2560, 5000])
def test_a_branch_closed_from_a_float32_result_with_its_bias(kernel_sets, dtype, d):
    ops, dt = kernel_sets[dtype], DTYPES[dtype]
    ref = TorchKernels(dt, DEV)
    g = torch.Generator(device="cpu").manual_seed(d)
    y = torch.randn(9, d, generator=g).to(DEV)
    bias, gain, nxt = [(0.5 + torch.rand(d, generator=g)).to(DEV) for _ in range(3)]
    base = torch.randn(9, d, generator=g).to(DEV)
    for yb in (bias, None):
        for yy in (y, y.to(dt)):
            r1, r2 = base.clone(), base.clone()
            a = ops.gated_norm_add(r1, yy, None, None, gain, 1e-5, 0.8, nxt, 1e-6, y_bias=yb)
            b = ref.gated_norm_add(r2, yy, None, None, gain, 1e-5, 0.8, nxt, 1e-6, y_bias=yb)
            torch.testing.assert_close(r1.cpu(), r2.cpu(), atol=2e-5, rtol=2e-5)
            _close(a, b, dtype, "the next norm's rows")


# ---- the models, cut in every way ------------------------------------------------------------------------------
def judged_in_bfloat16(got, want, rounded, what):
    """A request in bfloat16 against what rounding alone does to it, which the stand-in kernels in bfloat16 on the CPU
    say (they round where the HIP kernels round): within three times that for nine rows in ten (no fault of a window,
    a state, a page or a kernel keeps that), and for the worst row with room for a choice of experts that hangs on
    less than bfloat16 resolves and falls the other way."""
    mine, noise = row_errors(got.cpu(), want), row_errors(rounded, want)
    assert float(mine.max()) <= 3 * float(noise.max()) + 0.6, f"{what}: {float(mine.max()):.3g} against {float(noise.max()):.3g}"
    if mine.numel() >= 10:
        nine = int(0.9 * mine.numel())
        a, b = float(mine.kthvalue(nine).values), float(noise.kthvalue(nine).values)
        assert a <= 3 * b + 0.03, f"{what}, nine rows in ten: {a:.3g} against {b:.3g}"


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(MODELS))
def test_cuts_match_the_plain_model(folders, kernel_sets, name, cut, dtype):
    cfg = MODELS[name]
    prompts = random_prompts([3, 41, 70, 26, 1, 58], cfg["vocab"], seed=7)
    pool = dict(num_blocks=4 * (-(-72 // BLOCK[name]))) if cut == "mixed" else {}
    if dtype == "float32":
        check_trace(folders[name], kernel_sets[dtype], prompts, CUTS[cut](prompts), TOL[dtype], block_size=BLOCK[name], max_len=128,
                    what=f"{name} {cut} {dtype}", graphs=4 if cut in ("tail", "mixed") else 0, **pool)
        return
    runner = make_runner(folders[name], kernel_sets[dtype], max_rows=4, max_len=128, block_size=BLOCK[name], **pool)
    if cut in ("tail", "mixed"):
        runner.enable_graphs(4)
    got = replay(runner, CUTS[cut](prompts))
    rounded = replay(make_runner(folders[name], TorchKernels(torch.bfloat16, "cpu"), max_rows=4, max_len=128, block_size=BLOCK[name], **pool),
                     CUTS[cut](prompts))
    want = oracle(folders[name], prompts)
    for i in range(len(prompts)):
        judged_in_bfloat16(got[f"r{i}"], want[i], rounded[f"r{i}"], f"{name} {cut} request {i}")
    assert runner.cache.open_rows == []


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("seed", range(24))
def test_drawn_configurations(tmp_path, kernel_sets, seed, dtype):
    """Configurations drawn from everything config.json can say, each under one way of cutting its requests,
    captured decode steps included. Such models can be touchy (a width of 24, a sharp softmax, experts chosen by a
    hair): in bfloat16 a request is judged against what rounding alone does to it, which the stand-in kernels in
    bfloat16 on the CPU say (they round where the HIP kernels round): within three times that, per request, for
    nine rows in ten, and for the worst row unless a choice of experts fell the other way."""
    cfg = drawn_model(seed)
    folder = write_model(tmp_path / "m", cfg, seed=100 + seed)
    prompts = random_prompts([23, 1, 40, 9], cfg["vocab"], seed=seed)
    block = [2, 4, 16][seed % 3]
    cut = CUTS[["mixed", "portions", "tail"][seed % 3]]
    runner = make_runner(folder, kernel_sets[dtype], max_rows=4, max_len=64, block_size=block)
    if seed % 2:
        runner.enable_graphs(4)
    got = replay(runner, cut(prompts))
    want = oracle(folder, prompts)
    if dtype == "float32":
        for i in range(len(prompts)):
            compare(got[f"r{i}"], want[i], 1e-3, f"drawn {seed} {dtype} request {i}")
        return
    rounded = replay(make_runner(folder, TorchKernels(torch.bfloat16, "cpu"), max_rows=4, max_len=64, block_size=block), cut(prompts))
    for i in range(len(prompts)):
        judged_in_bfloat16(got[f"r{i}"], want[i], rounded[f"r{i}"], f"drawn {seed} request {i}")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_a_wider_model_with_long_prompts(tmp_path, kernel_sets, dtype):
    """Width 320, five layers, maps of 80 beside values of 48, a memory of 64 x 96, keys that are values of 64, a
    layer on another's cache behind a narrower window, prompts of up to 700 tokens: decoded at the end, mixed, and in
    portions of 2 to 200 tokens, through captured decode steps; long portions go to the prompt kernel on the
    matrix cores where the score terms allow."""
    position = rot(40, 40000.0, (3.0, 256, 16.0, 1.0))
    cfg = model(320, 500, [differential(10, 5, 80, 48, size=100, keep=7, rotation=position, diff=0.4, scale=0.1),
                           memory(5, 64, 96, 15.0),
                           differential(10, 5, 80, 48, size=37, keep=20, rotation=position, diff=0.7, scale=0.15, kv_from=0),
                           keyed(8, 2, 64, rot(64, 1e6, (8.0, 512, 32.0, 1.0)), scale=2.0, softcap=30.0),
                           memory(2, 128, 32, 4.0)],
                [moe(16, 4, 96, count=4, keep=2, scale=1.3, shared=200), moe(6, 2, 100), None, moe(8, 1, 64, count=2, keep=1, shared=64),
                 moe(4, 2, 320, scale=2.0)], embedding=4.0)
    folder = write_model(tmp_path / "m", cfg, seed=5)
    prompts = random_prompts([700, 333, 64, 150], cfg["vocab"], seed=6)
    want = oracle(folder, prompts)
    for name, steps in (("tail", trace_tail_decode(prompts, 40)), ("mixed", trace_mixed(prompts, seed=7)),
                        ("portions", trace_portions(prompts, seed=8, sizes=(2, 3, 64, 65, 128, 200)))):
        runner = make_runner(folder, kernel_sets[dtype], max_rows=4, max_len=768, block_size=16, num_blocks=4 * 48)
        runner.enable_graphs(4)
        got = replay(runner, steps)
        for i in range(len(prompts)):
            compare(got[f"r{i}"], want[i], TOL[dtype], f"{name} {dtype} request {i}")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_a_model_of_a_thousand_columns(tmp_path, kernel_sets, dtype):
    """Width 1,024 and heads of 128: matrices large enough for the products' other forms (weights read by tile, the
    sweeps, the library beyond 16 rows, the experts' large tiles), a state of 128 x 128, two maps of 128 over values of
    64, prompts of up to 300 tokens decoded at the end and mixed, through captured decode steps."""
    position = rot(64, 500000.0, (8.0, 4096, 16.0, 2.0))
    cfg = model(1024, 2000, [memory(4, 128, 128, 18.0),
                             differential(4, 2, 128, 64, size=64, keep=6, rotation=position, diff=0.35, scale=0.09),
                             keyed(8, 4, 128, rot(128, 1e6, (4.0, 1024, 16.0, 1.0)), scale=6.0, softcap=20.0),
                             differential(4, 2, 128, 64, size=150, keep=2, rotation=position, diff=0.6, scale=0.09, kv_from=1)],
                [moe(8, 2, 512, count=4, keep=2, scale=1.8, shared=768), moe(4, 1, 1024), None, moe(8, 3, 256, count=2, keep=2, shared=256)],
                embedding=10.0)
    folder = write_model(tmp_path / "m", cfg, seed=9)
    prompts = random_prompts([300, 120, 33], cfg["vocab"], seed=10)
    want = oracle(folder, prompts)
    for name, steps in (("tail", trace_tail_decode(prompts, 24)), ("mixed", trace_mixed(prompts, seed=11))):
        runner = make_runner(folder, kernel_sets[dtype], max_rows=4, max_len=320, block_size=16)
        runner.enable_graphs(4)
        got = replay(runner, steps)
        if dtype == "float32":
            for i in range(len(prompts)):
                compare(got[f"r{i}"], want[i], TOL[dtype], f"{name} {dtype} request {i}")
        else:
            rounded = replay(make_runner(folder, TorchKernels(torch.bfloat16, "cpu"), max_rows=4, max_len=320, block_size=16), steps)
            for i in range(len(prompts)):
                judged_in_bfloat16(got[f"r{i}"], want[i], rounded[f"r{i}"], f"{name} request {i}")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_edges_and_long_decoding(tmp_path, kernel_sets, dtype):
    """A window of 6 with 3 kept tokens, read again by a layer behind a window of 4 with 5 kept (in float32 under a
    sharp softmax, so the key at an edge often carries the weight; in bfloat16 a flatter one, where rounding moves
    little), pages of 4, 150 tokens decoded one by one from captured steps: the windows pass over decoded tokens,
    pages behind them come back, the first stay."""
    scale = 2.0 if dtype == "float32" else 0.4
    position = rot(8, 1000.0, RAMP)
    cfg = model(48, 50, [differential(2, 1, 16, 8, size=6, keep=3, rotation=position, diff=0.3, scale=scale),
                         differential(2, 1, 16, 8, size=4, keep=5, rotation=position, diff=0.6, scale=scale, kv_from=0),
                         memory(2, 16, 24, 9.0)],
                [moe(4, 2, 32, shared=24), None, None], embedding=2.0)
    folder = write_model(tmp_path / "m", cfg, seed=21)
    prompts = random_prompts([160], cfg["vocab"], seed=22)
    want = oracle(folder, prompts)
    runner = make_runner(folder, kernel_sets[dtype], max_rows=2, max_len=192, block_size=4, num_blocks=8)
    runner.enable_graphs(2)
    got = replay(runner, trace_tail_decode(prompts, 150))
    compare(got["r0"], want[0], TOL[dtype], "decoded behind the windows")
    # the test sees an edge that is one off: the plain model with such constants is far outside the limits
    pcfg, w = read_folder(folder)
    for layer, key, other in ((0, "size", 7), (0, "keep_first", 2), (1, "size", 5), (1, "keep_first", 6)):
        mask = pcfg["layers"][layer]["mixer"]["mask"]
        was, mask[key] = mask[key], other
        with pytest.raises(AssertionError):
            compare(plain.forward(pcfg, w, prompts[0]).float(), want[0], TOL[dtype])
        mask[key] = was


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_captured_decode_steps_equal_eager_ones(folders, kernel_sets, dtype):
    cfg = MODELS["A"]
    prompts = random_prompts([30, 45, 9], cfg["vocab"], seed=31)
    steps = trace_mixed(prompts, seed=32, max_live=3, prefill_frac=0.3)
    eager = replay(make_runner(folders["A"], kernel_sets[dtype], max_len=64, block_size=4), steps)
    runner = make_runner(folders["A"], kernel_sets[dtype], max_len=64, block_size=4)
    runner.enable_graphs(4)
    assert runner.graphs_refused is None and runner.model.capturable
    captured = replay(runner, steps)
    assert runner._graphs, "no decode step was captured"
    for rid in eager:
        torch.testing.assert_close(captured[rid], eager[rid], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("name", ["A", "memory", "B"])
def test_greedy_generation_through_the_engine(folders, name):
    """``Engine(folder)`` finds the model class by config.json; float32 greedy tokens are the plain model's,
    with more requests than rows, so rows, states and pages are used again."""
    from socrates_amd.engine import Engine
    cfg, w = read_folder(folders[name])
    prompts = random_prompts([5, 17, 33, 2, 21, 11], cfg["vocab"], seed=41)
    want = [plain.greedy(cfg, w, p, 8) for p in prompts]
    engine = Engine(str(folders[name]), device=DEV, dtype=torch.float32, max_batch=3, max_len=64, max_new_tokens=8,
                    block_size=BLOCK[name], chunk=16)
    assert engine.generate(prompts, max_new_tokens=8) == want
    engine.cache.check()


def test_command_line(tmp_path, folders):
    """``python -m socrates_amd.generate`` on a model folder, and with ``--random-weights`` on a configuration alone
    (it writes a seeded random model into --model): float32 greedy tokens are the plain model's."""
    cfg, w = read_folder(folders["A"])
    prompts = random_prompts([5, 17], cfg["vocab"], seed=2)
    want = [plain.greedy(cfg, w, p, 5) for p in prompts]
    cmd = [sys.executable, "-m", "socrates_amd.generate", "--model", str(folders["A"]), "--dtype", "float32",
           "--max-new-tokens", "5", "--max-len", "64", "--max-batch", "2", "--block-size", "4"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(ROOT))
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().split("\n")
    shown = [l for i, l in enumerate(lines) if i > 0 and lines[i - 1].startswith("> ")]
    assert shown == [" ".join(map(str, x)) for x in want]
    (tmp_path / "config.json").write_text(json.dumps(MODELS["B"]))
    made = tmp_path / "made"
    cmd = [sys.executable, "-m", "socrates_amd.generate", "--model", str(made), "--random-weights", str(tmp_path / "config.json"),
           "--seed", "4", "--dtype", "float32", "--max-new-tokens", "4", "--max-len", "64", "--max-batch", "2",
           "--prompt-ids", "7,100,12,5,9"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(ROOT))
    assert proc.returncode == 0, proc.stderr[-2000:]
    cfg, w = read_folder(made)
    assert cfg == MODELS["B"]
    lines = proc.stdout.strip().split("\n")
    shown = [l for i, l in enumerate(lines) if i > 0 and lines[i - 1].startswith("> ")]
    assert shown == [" ".join(map(str, plain.greedy(cfg, w, [7, 100, 12, 5, 9], 4)))]


def test_trace_runner_on_a_model_folder(tmp_path, folders):
    cfg = MODELS["A"]
    prompts = random_prompts([70, 33, 100, 12, 64], cfg["vocab"], seed=51)
    want = oracle(folders["A"], prompts)
    steps = trace_mixed(prompts, seed=52)
    lines, wanted, fed = [], [], {}
    for n, (entries, ends) in enumerate(steps):
        lines.append(json.dumps({"step": n, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in entries], "end": ends}))
        here = []
        for r, t, w in entries:
            here.append((int(r[1:]), [fed.get(r, 0) + j for j in w]))
            fed[r] = fed.get(r, 0) + len(t)
        wanted.append(here)
    max_tokens = sum(-(-len(p) // 64) * 64 for p in sorted(prompts, key=len)[-4:])
    for dtype in DTYPES:
        out = tmp_path / dtype
        proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folders["A"]), "--dtype", dtype,
                               "--out", str(out), "--max-tokens", str(max_tokens)], input="\n".join(lines) + "\n",
                              capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert proc.stdout.split("\n")[:-1] == [f"done {i}" for i in range(len(lines))]
        for n, here in enumerate(wanted):
            rows = sum(len(pos) for _, pos in here)
            if rows:
                got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(rows, cfg["vocab"]).copy())
                compare(got, torch.cat([want[i][pos] for i, pos in here]), TOL[dtype], f"step {n} {dtype}")
