"""Muzasun on the GPU against the plain implementation (``plain/muzasun_plain.py``): kernels and mechanisms alone, then
whole models through the step function (whole prompts, single tokens, portions down to two tokens, mixed batches,
slots and pages that are used again, far keys, page borders), and greedy generation through the engine.

The plain implementation runs whole sequences in float64; every check feeds the engine's logits at all positions of a
request, however they were cut into steps, against its logits of the whole sequence.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import muzasun_helpers as M
from helpers import assert_tokens_follow_plain, rel_err
from plain import muzasun_plain as P

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 0.1}     # of a position's largest logit; observed 3e-5 and 0.05


def open_runner(folder, dtype, pages=64, page=8, slots=4):
    from vipera_rs_amd.engine.runner import ModelRunner

    return ModelRunner.from_folder(folder, dtype=dtype, block_size=page, num_blocks=pages, num_slots=slots)


def replay(runner, requests, plan, keep=()):
    """Run ``plan`` (steps of (request, tokens) pairs) and return every request's logits at all its positions.
    A request gives back its pages and slot when its last token has run, unless it is in ``keep``."""
    from vipera_rs_amd.engine.batch import StepEntry

    at = {r: 0 for r in requests}
    rows = {r: [] for r in requests}
    for step in plan:
        entries = []
        for r, size in step:
            runner.cache.reserve(r, at[r], at[r] + size)
            entries.append(StepEntry(r, at[r], requests[r][at[r]:at[r] + size], list(range(size))))
        logits = runner.step(entries).float().cpu().numpy()
        row = 0
        for r, size in step:
            rows[r].append(logits[row:row + size])
            row += size
            at[r] += size
            runner.cache.advance(r, at[r])
            if at[r] == len(requests[r]) and r not in keep:
                runner.cache.release(r)
    return {r: np.concatenate(v) for r, v in rows.items() if v}


def check(got, want, tol, label=""):
    """Position by position, so that one wrong token cannot hide among many right ones.  In 32-bit every position
    must hold.  In bfloat16 a router's close call may fall the other way than in float64 and move one position's
    logits (and, through the recurrent layers' state, a few after it) by more than rounding: there one position in
    twenty may be over, which a fault of a page, a slot or a state (whole runs of positions) still exceeds."""
    strict = tol < 1e-3
    over, total = [], 0
    for r in got:
        n = got[r].shape[0]
        assert want[r].shape[0] == n
        for t in range(n):
            err = rel_err(got[r][t], want[r][t])
            total += 1
            if not err < tol:
                assert not strict, f"{label}: request {r}, position {t} of {n}: relative error {err:.3g}"
                over.append((r, t, round(err, 3)))
    assert len(over) <= total // 20, f"{label}: {len(over)} of {total} positions are over {tol}: {over[:8]}"


def tokens_for(cfg, w, count, seed):
    return M.clear_tokens(cfg, w, count, seed)


def portions(total, sizes):
    out, k = [], 0
    while total:
        size = min(sizes[k % len(sizes)], total)
        out.append(size)
        total -= size
        k += 1
    return out


# --- kernels alone ------------------------------------------------------------------------------------------------
def test_routing_weighs_by_the_sigmoid_of_the_chosen_logits():
    from vipera_rs_amd.ops import kernels

    logits = torch.tensor([[0.5, 2.0, 1.9, -1.0, 1.8, 0.0], [1.0, -3.0, 1.0, 0.0, 1.0, 0.5], [-5.0] * 6])
    many = torch.randn((40, 6), generator=torch.Generator().manual_seed(1))
    for z, top in ((logits, 3), (many, 2), (many, 6)):
        tokens, experts = z.shape
        pairs = tokens * top
        ids = torch.empty(pairs, dtype=torch.int32, device="cuda")
        order, weights = torch.empty_like(ids), torch.empty(pairs, device="cuda")
        offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
        tiles = torch.empty(2 * kernels.moe_max_tiles(pairs, experts), dtype=torch.int32, device="cuda")
        count = torch.empty(1, dtype=torch.int32, device="cuda")
        kernels.moe_route(z.cuda(), top, ids, weights, offsets, order, tiles, count, all_scores="sigmoid")
        ids, weights = ids.view(tokens, top).cpu(), weights.view(tokens, top).cpu()
        scores = P.sigmoid(z.double().numpy())
        for t in range(tokens):
            want = P.route(scores[t], top)
            assert ids[t].tolist() == want                  # the lower id among equals
            assert np.allclose(weights[t].numpy(), scores[t][want], atol=1e-6)       # not renormalized
        assert sorted(order.cpu().tolist()) == list(range(pairs))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_normed_one_by_one_and_values_blended(dtype):
    from vipera_rs_amd.ops import kernels

    rng = np.random.default_rng(3)
    tokens, heads, kv_heads, dim, vdim, padded = 9, 3, 2, 10, 14, 16
    proj = rng.standard_normal((tokens, (heads + kv_heads) * dim + kv_heads * vdim + 5))
    first = rng.standard_normal((tokens, kv_heads * vdim + 3))
    qw, kw, lam = 1 + 0.1 * rng.standard_normal(dim), 1 + 0.1 * rng.standard_normal(dim), 0.37
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    out = torch.full((tokens, (heads + 2 * kv_heads) * padded), float("nan"), dtype=dtype, device="cuda")
    kernels.head_norm_pack(dev(proj), dev(qw), dev(kw), 1e-5, heads, kv_heads, dim, vdim, padded, out,
                           dev(first)[:, :kv_heads * vdim], dev([lam]))
    got = out.float().cpu().numpy().reshape(tokens, heads + 2 * kv_heads, padded)
    q = proj[:, :heads * dim].reshape(tokens, heads, dim)
    k = proj[:, heads * dim:(heads + kv_heads) * dim].reshape(tokens, kv_heads, dim)
    v = proj[:, (heads + kv_heads) * dim:(heads + kv_heads) * dim + kv_heads * vdim].reshape(tokens, kv_heads, vdim)
    v = (1 - lam) * v + lam * first[:, :kv_heads * vdim].reshape(tokens, kv_heads, vdim)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert rel_err(got[:, :heads, :dim], P.over_rms(q, 1e-5) * qw) < tol
    assert rel_err(got[:, heads:heads + kv_heads, :dim], P.over_rms(k, 1e-5) * kw) < tol
    assert rel_err(got[:, heads + kv_heads:, :vdim], v) < tol
    assert not got[:, :heads + kv_heads, dim:].any() and not got[:, heads + kv_heads:, vdim:].any()     # zeros in the padding


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows, width", [(7, 50), (5, 1100), (3, 4700), (300, 520)])
def test_two_norms_of_the_same_rows_in_one_launch(rows, width, dtype):
    """Few rows are spread over several workgroups each (a last part that is not full, more columns than one pass of
    all parts covers); many rows are a workgroup each."""
    from vipera_rs_amd.ops import kernels

    rng = np.random.default_rng(4)
    x = rng.standard_normal((rows, width)) * 2.0
    dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device="cuda")
    norms = [(np.array([0.7 + k]), 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)) for k in range(2)]
    outs = [torch.empty((rows, width), dtype=dtype, device="cuda") for _ in range(2)]
    kernels.dyt_pair(dev(x), *[tuple(dev(t) for t in norm) for norm in norms], *outs)
    for (alpha, weight, bias), out in zip(norms, outs):
        single = torch.empty_like(out)
        kernels.dyt(dev(x), dev(alpha), dev(weight), dev(bias), single)
        assert torch.equal(out, single)                  # the same bits as the norm alone
        assert rel_err(out.float().cpu().numpy(), np.tanh(alpha * x) * weight + bias) < (1e-6 if dtype == torch.float32 else 1e-2)


# --- each mechanism alone, as a model of one layer -------------------------------------------------------------------
ONE_LAYER = {
    # the matrix memory at every register layout of its two kernels (1 to 16 key channels a lane)
    "memory": M.single(M.memory(2, 16, 16)),
    "memory_three_odd_heads": M.single(M.memory(3, 10, 14, cap=4.0), width=48),
    "memory_one_wide_head": M.single(M.memory(1, 40, 20, cap=30.0), width=40),
    "memory_wider": M.single(M.memory(2, 72, 5), width=72),
    "memory_widest": M.single(M.memory(1, 136, 33), width=72),
    # the delta rule with a decay per key channel, likewise
    "delta": M.single(M.delta(4, 2, 16, 8, 4)),
    "delta_one_tap_odd": M.single(M.delta(2, 1, 10, 14, 1, ranks=(3, 7)), width=50),
    "delta_equal_heads": M.single(M.delta(2, 2, 24, 24, 2, ranks=(8, 8)), width=48),
    "delta_wider": M.single(M.delta(2, 1, 72, 40, 3), width=72),
    "delta_widest": M.single(M.delta(1, 1, 136, 20, 5, ranks=(16, 1)), width=72),
    # attention: values wider and narrower than keys and as wide; partial, full and no rotation; grouped heads
    "attention": M.single(M.attention(4, 2, 16, 24, rot_dims=8, base=1000.0, scale=0.3, v_mix=True)),
    "attention_narrow_values": M.single(M.attention(3, 1, 24, 8), width=48),
    "attention_no_rotation_odd": M.single(M.attention(2, 2, 10, 6, rot_dims=0, scale=0.4), width=50),
    "attention_equal_widths": M.single(M.attention(2, 1, 32, 32, rot_dims=16)),
    "attention_wide": M.single(M.attention(5, 5, 72, 136, rot_dims=32), width=136),
    # feed-forwards beside a small mixer
    "dense": M.single(M.memory(1, 8, 8), M.dense(56), width=48, mult=0.5),
    "experts": M.single(M.memory(1, 8, 8), M.moe(8, 3, 40, shared=24), width=48, mult=0.5),
    "experts_no_shared_top_one": M.single(M.memory(1, 8, 8), M.moe(5, 1, 18), width=50),
    "experts_all_chosen": M.single(M.memory(1, 8, 8), M.moe(3, 3, 24, shared=8), width=48, logit_scale=0.5),
    "experts_wide": M.single(M.memory(1, 8, 8), M.moe(8, 2, 160, shared=136), width=136),
}
LONG = {"experts_wide", "attention_wide"}       # a prompt of 330 tokens: several tiles per expert and per head


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ONE_LAYER))
def test_a_mechanism_alone_whole_prompt_then_single_tokens(tmp_path, name, dtype):
    cfg = ONE_LAYER[name]
    folder = M.make_folder(tmp_path / name, cfg, 11)
    plain_cfg, w = M.load_folder(folder)
    first = 330 if name in LONG else 45
    requests = {0: tokens_for(plain_cfg, w, first, 1), 1: tokens_for(plain_cfg, w, 30, 2)}
    want = {r: P.forward(plain_cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype)
    plan = [[(0, first)], [(1, 19)]] + [[(1, 1)]] * 11
    check(replay(runner, requests, plan), want, TOL[dtype], name)
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


def test_the_residual_after_every_layer(tmp_path):
    """32-bit, layer by layer: a fault shows in the layer that has it, not only in the logits."""
    folder = M.make_folder(tmp_path / "m1", M.M1, 21)
    plain_cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(M.M1["vocab"], 40, 5)
    residuals = []
    P.forward(plain_cfg, w, tokens, residuals)
    runner = open_runner(folder, "float32")
    seen = []
    for layer in runner.model.layers:
        def wrapped(x, *args, _forward=layer.forward, **kwargs):
            _forward(x, *args, **kwargs)
            seen.append(x.clone())
        layer.forward = wrapped
    replay(runner, {0: tokens}, [[(0, 40)]])
    assert len(seen) == len(residuals) == 5
    for index, (got, ref) in enumerate(zip(seen, residuals)):
        assert rel_err(got.cpu().numpy(), ref) < 1e-5, f"after layer {index} ({M.M1['layers'][index]['type']})"


def test_blended_values_are_what_later_layers_cache(tmp_path):
    """The test has teeth: the second blending layer's number moves the logits, and so would values of the wrong layer
    or token; then the engine holds to the plain implementation where half of every value comes from the first layer,
    in a prompt, in portions and token by token (the blended values come back out of the cache)."""
    cfg = M.config(61, 32, [M.attention(2, 2, 8, 12, v_mix=True), M.memory(1, 8, 8), M.attention(4, 2, 8, 12, rot_dims=4, v_mix=True)],
                   [None, None, None], mult=1.0)

    def half(tensors):
        tensors["l2.mix.vmix"] = torch.tensor(0.5, dtype=torch.bfloat16)
    folder = M.make_folder(tmp_path / "blend", cfg, 5, edit=half)
    cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(61, 50, 3)
    want = P.forward(cfg, w, tokens)
    none = dict(w)
    none["l2.mix.vmix"] = np.float64(0.0)
    assert rel_err(P.forward(cfg, none, tokens), want) > 0.05
    for dtype in ("float32", "bfloat16"):
        runner = open_runner(folder, dtype)
        for plan in ([[(0, 50)]], [[(0, n)] for n in portions(50, [7, 2, 1, 19])], [[(0, 1)]] * 50):
            check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "blended values")


# --- whole models through the step function ------------------------------------------------------------------------
@pytest.fixture(scope="module")
def m1(tmp_path_factory):
    folder = M.make_folder(tmp_path_factory.mktemp("m1"), M.M1, 31)
    return (folder,) + M.load_folder(folder)


@pytest.fixture(scope="module")
def m2(tmp_path_factory):
    folder = M.make_folder(tmp_path_factory.mktemp("m2"), M.M2, 32)
    return (folder,) + M.load_folder(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["m1", "m2"])
def test_token_by_token_equals_the_whole_prompt(request, which, dtype):
    folder, cfg, w = request.getfixturevalue(which)
    tokens = tokens_for(cfg, w, 70, 7)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype, page=4 if which == "m2" else 8, pages=128 if which == "m2" else 64)
    whole = replay(runner, {0: tokens}, [[(0, 70)]])
    check(whole, want, TOL[dtype], "whole")
    single = replay(runner, {0: tokens}, [[(0, 1)]] * 70)      # long decoding from the very first token
    check(single, want, TOL[dtype], "token by token")
    if dtype == "float32":   # the two ways differ by rounding only
        assert rel_err(single[0], whole[0].astype(np.float64)) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 2, 5], [13, 1, 8], [16, 2], [64, 7]])
def test_portions_of_a_prompt(m1, sizes, dtype):
    """Portions cut inside pages (8), at their borders, inside the convolution's reach (3 taps) and inside the
    recurrences' blocks of 16 tokens."""
    folder, cfg, w = m1
    tokens = tokens_for(cfg, w, 83, 9)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype)
    plan = [[(0, n)] for n in portions(83, sizes)]
    check(replay(runner, {0: tokens}, plan), want, TOL[dtype], f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["m1", "m2"])
def test_a_mixed_batch_equals_each_request_alone(request, which, dtype):
    """Up to four live requests of unequal lengths: portions of some beside single tokens of others; requests end and
    later ones take their slots and pages; the pool holds less than all requests together."""
    folder, cfg, w = request.getfixturevalue(which)
    lengths = {0: 61, 1: 9, 2: 40, 3: 1, 4: 33, 5: 26, 6: 2}
    requests = {r: tokens_for(cfg, w, n, 40 + r) for r, n in lengths.items()}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    plan = [[(0, 20), (1, 2), (2, 7)], [(0, 1), (1, 7), (2, 2), (3, 1)], [(0, 17), (2, 1), (4, 30)],
            [(0, 2), (2, 30), (4, 1), (5, 5)], [(0, 1), (4, 1), (5, 2), (6, 2)], [(0, 20), (4, 1), (5, 19)]]
    runner = open_runner(folder, dtype, pages=22, page=8, slots=4)    # 176 positions for 172 tokens in all
    got = replay(runner, requests, plan)
    assert {r: v.shape[0] for r, v in got.items()} == lengths
    check(got, want, TOL[dtype], "mixed")
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_and_pages_that_are_used_again_start_clean(m1, dtype):
    """One slot and few pages: every request runs in the state row and the pages the one before it left full."""
    folder, cfg, w = m1
    runner = open_runner(folder, dtype, pages=9, page=8, slots=1)
    for r, (n, cut) in enumerate([(60, [60]), (41, [5, 2, 30, 1, 1, 1, 1]), (17, [1] * 17), (64, [33, 31])]):
        tokens = tokens_for(cfg, w, n, 70 + r)
        got = replay(runner, {r: tokens}, [[(r, size)] for size in cut])
        check(got, {r: P.forward(cfg, w, tokens)}, TOL[dtype], f"request {r} in the used slot")
        assert runner.cache.slot(r) == -1 and runner.cache.free_slots() == 1


def test_state_rows_full_of_nan_do_not_reach_a_new_request(m2):
    """A slot's rows may hold anything when a request takes it: every recurrence starts from zeros at position 0."""
    folder, cfg, w = m2
    runner = open_runner(folder, "float32", slots=2)
    for state in runner.storage.state:
        if state is not None:
            state.fill_(float("nan"))
    tokens = tokens_for(cfg, w, 21, 4)
    want = {0: P.forward(cfg, w, tokens)}
    check(replay(runner, {0: tokens}, [[(0, 1)], [(0, 12)], [(0, 1)], [(0, 7)]]), want, TOL["float32"], "NaN rows")


def test_a_model_without_attention_keeps_no_pages(tmp_path):
    cfg = M.config(61, 32, [M.memory(2, 8, 8), M.delta(1, 1, 16, 8, 2)], [M.dense(24), None], mult=1.5)
    folder = M.make_folder(tmp_path / "flat", cfg, 4)
    cfg, w = M.load_folder(folder)
    requests = {0: M.tokens_of(61, 50, 1), 1: M.tokens_of(61, 12, 2)}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, "float32", pages=2, slots=2)
    plan = [[(0, 30), (1, 2)], [(0, 1), (1, 9)], [(0, 19), (1, 1)]]
    check(replay(runner, requests, plan), want, TOL["float32"], "no attention")


# --- far keys, page borders, long memory ------------------------------------------------------------------------------
SHARP_TOL = {"float32": 1e-4, "bfloat16": 8e-2}    # peaked attention weights amplify the rounding of queries and keys


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dtype):
    """Peaked attention (the norms' weights scaled up): a late query puts most of its weight on single keys anywhere
    among its visible positions, hundreds of positions and many pages back, so a key that is lost or misplaced shows;
    portions end on page borders, one before and one behind them."""
    cfg = M.single(M.attention(2, 1, 16, 24, rot_dims=8, scale=0.25), vocab=61)
    folder = M.make_folder(tmp_path / "far", cfg, 8, sharp=2.0)
    cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(cfg["vocab"], 400, 17)
    want = P.forward(cfg, w, tokens)
    # the test has teeth: without its first hundred positions a late token's logits move clearly
    cut = P.forward(cfg, w, tokens[100:])
    assert sum(rel_err(cut[t - 100], want[t]) > 0.1 for t in range(300, 400)) > 50
    runner = open_runner(folder, dtype, pages=60, page=16)
    for plan in ([[(0, 400)]], [[(0, 340)]] + [[(0, 1)]] * 60, [[(0, n)] for n in portions(400, [127, 2, 64, 33])],
                 [[(0, 16)], [(0, 15)], [(0, 17)], [(0, 208)]] + [[(0, 1)]] * 12 + [[(0, 132)]]):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], "far key")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim, vdim", [(64, 64), (128, 96)])
def test_a_long_prompt_on_the_prompt_kernels_of_full_head_widths(tmp_path, dim, vdim, dtype):
    cfg = M.single(M.attention(4, 2, dim, vdim, rot_dims=dim // 2), vocab=61, width=64)
    folder = M.make_folder(tmp_path / "long", cfg, 12)
    cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(cfg["vocab"], 1300, 23)
    want = P.forward(cfg, w, tokens)
    runner = open_runner(folder, dtype, pages=90, page=16)
    for plan in ([[(0, 1300)]], [[(0, 700)], [(0, 590)]] + [[(0, 1)]] * 10):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "long prompt")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["memory", "delta"])
def test_a_state_that_forgets_slowly_remembers_the_first_tokens(tmp_path, kind, dtype):
    """Forget gates near one (decays near one): after 300 tokens, in pieces, the first tokens still weigh in the output,
    which a state that is lost or cleared between steps would not show."""
    layer = M.memory(2, 16, 16) if kind == "memory" else M.delta(2, 1, 16, 16, 3)
    cfg = M.single(layer, vocab=61, width=32)

    def slow(tensors):
        if kind == "memory":
            tensors["l0.mix.f.b"] = torch.full((2,), 6.0, dtype=torch.bfloat16)
            tensors["l0.mix.i.b"] = torch.full((2,), -2.0, dtype=torch.bfloat16)
        else:
            tensors["l0.mix.dt_bias"] = torch.full((32,), -6.0, dtype=torch.bfloat16)
            tensors["l0.mix.A_log"] = torch.full((2,), -1.0, dtype=torch.bfloat16)
    folder = M.make_folder(tmp_path / "slow", cfg, 9, edit=slow)
    cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(cfg["vocab"], 300, 19)
    want = P.forward(cfg, w, tokens)
    forgot = P.forward(cfg, w, tokens[150:])
    assert rel_err(forgot[-20:], want[-20:]) > 0.05            # the first half matters to the end
    runner = open_runner(folder, dtype)
    for plan in ([[(0, 300)]], [[(0, n)] for n in portions(300, [150, 1, 1, 2, 97])], [[(0, 260)]] + [[(0, 1)]] * 40):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "slow state")


def test_gates_at_their_caps(tmp_path):
    """Input gates far above the cap and forget gates far below: the running maximum and the floor of the denominator
    carry the scale, in a prompt and token by token."""
    cfg = M.single(M.memory(2, 16, 8, cap=3.0), vocab=61, width=32)

    def extreme(tensors):
        tensors["l0.mix.i.b"] = torch.tensor([40.0, -40.0], dtype=torch.bfloat16)
        tensors["l0.mix.f.b"] = torch.tensor([-40.0, 40.0], dtype=torch.bfloat16)
    folder = M.make_folder(tmp_path / "caps", cfg, 2, edit=extreme)
    cfg, w = M.load_folder(folder)
    tokens = M.tokens_of(61, 60, 6)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, "float32")
    for plan in ([[(0, 60)]], [[(0, 1)]] * 60, [[(0, 17)], [(0, 2)], [(0, 41)]]):
        check(replay(runner, {0: tokens}, plan), want, TOL["float32"], "gates at their caps")


def test_the_first_tokens_of_a_sequence(m1):
    """Positions 0 to 4 one by one and as a portion: nothing before position 0 exists (no state, zeros before the
    convolution's start, a running maximum of 0)."""
    folder, cfg, w = m1
    runner = open_runner(folder, "float32")
    for n in (1, 2, 3, 5):
        tokens = M.tokens_of(cfg["vocab"], n, 90 + n)
        want = {0: P.forward(cfg, w, tokens)}
        check(replay(runner, {0: tokens}, [[(0, n)]]), want, TOL["float32"], f"{n} tokens at once")
        check(replay(runner, {0: tokens}, [[(0, 1)]] * n), want, TOL["float32"], f"{n} tokens one by one")


# --- the engine: scheduler, sampling, captured steps ------------------------------------------------------------------
@pytest.mark.parametrize("dtype, graphs, pipelined", [("float32", False, False), ("float32", True, False),
                                                      ("float32", True, True), ("bfloat16", True, True)])
def test_greedy_generation_through_the_engine(m1, dtype, graphs, pipelined):
    from vipera_rs_amd import Engine

    folder, cfg, w = m1
    prompts = [M.tokens_of(cfg["vocab"], n, 60 + n) for n in (5, 37, 18, 2, 23)]
    new_tokens = 24
    engine = Engine(folder, dtype=dtype, block_size=8, num_blocks=40, max_num_seqs=3, chunk_size=16,
                    max_num_batched_tokens=32, max_model_len=128, use_graphs=graphs, pipelined=pipelined)
    got = engine.generate(prompts, max_new_tokens=new_tokens)
    clear = followed = 0
    for prompt, generation in zip(prompts, got):
        assert len(generation.tokens) == new_tokens
        logits = P.forward(cfg, w, prompt + generation.tokens[:-1])
        if dtype == "float32":
            clear += assert_tokens_follow_plain(logits, len(prompt), generation.tokens, 2.5e-5, f"prompt of {len(prompt)}")
            continue
        # bfloat16: where the plain implementation's best token leads by a fifth of the largest logit, the engine's
        # token should be that one; a router's close call may move single positions by more (their tokens are the
        # engine's own, not chosen for clear routing), so a few may differ
        for k, token in enumerate(generation.tokens):
            row = logits[len(prompt) - 1 + k]
            order = np.argsort(row)
            if row[order[-1]] - row[order[-2]] > 0.2 * np.max(np.abs(row)):
                clear += 1
                followed += int(token) == int(order[-1])
    if dtype == "float32":
        assert clear >= 100, clear
    else:
        assert clear >= 15 and followed >= 0.9 * clear, (clear, followed)
    if graphs:
        assert engine.runner.graphs.replays > 0
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_the_command_line_generates(m2):
    """``bin/vipera generate`` on a Muzasun folder: the model is found by its configuration and run through the engine."""
    folder, cfg, w = m2
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = M.tokens_of(cfg["vocab"], 11, 3)
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "vipera"), "generate", folder, "--prompt-ids",
                           " ".join(str(t) for t in prompt), "--max-tokens", "8", "--dtype", "float32", "--json"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    report = json.loads(done.stdout)
    assert report["prompt_tokens"] == 11 and report["generated_tokens"] == 8
    logits = P.forward(cfg, w, prompt + report["tokens"][:-1])
    assert assert_tokens_follow_plain(logits, len(prompt), report["tokens"], 2.5e-5, "command line") >= 4


def test_the_trace_runner_replays_a_schedule(tmp_path, m1):
    """``bin/trace_run`` on a Muzasun folder: four slots, pages for the live requests only."""
    folder, cfg, w = m1
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = M.tokens_of(cfg["vocab"], 50, 1), M.tokens_of(cfg["vocab"], 20, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[30:32], "want": []}, {"id": "b", "tokens": b[:19], "want": [18]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[19:], "want": [0]}, {"id": "a", "tokens": a[32:], "want": [17]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = P.forward(cfg, w, a), P.forward(cfg, w, b)
    rows = {0: [wa[0], wa[29]], 1: [wb[18]], 2: [wb[19], wa[49]]}
    for step, want in rows.items():
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(want), cfg["vocab"])
        assert rel_err(got, np.stack(want)) < TOL["float32"]
