"""Lurirax on the GPU against the plain implementation (``plain/lurirax_plain.py``): kernels and mechanisms alone, then
whole models through the step function (whole prompts, single tokens, portions down to two tokens, mixed batches,
slots and pages that are used again, far keys, the edges of windows, chunks and kept first positions, page borders),
and greedy generation through the engine.

The plain implementation runs whole sequences in float64; every check feeds the engine's logits at all positions of a
request, however they were cut into steps, against its logits of the whole sequence.
"""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import lurirax_helpers as L
from helpers import assert_tokens_follow_plain, rel_err
from plain import lurirax_plain as P

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 0.1}     # of a position's largest logit


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
    logits (and, through retention's state, a few after it) by more than rounding: there one position in twenty may
    be over, which a fault of a page, a slot or a state (whole runs of positions) still exceeds."""
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


def portions(total, sizes):
    out, k = [], 0
    while total:
        size = min(sizes[k % len(sizes)], total)
        out.append(size)
        total -= size
        k += 1
    return out


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).cuda()


# --- kernels alone ------------------------------------------------------------------------------------------------
def test_routing_steered_by_a_correction():
    from vipera_rs_amd.ops import kernels

    logits = torch.tensor([[3.0, 2.0, 1.0, 0.0], [0.0, 0.0, 0.0, 0.0], [-4.0, 4.0, 4.0, -4.0]])
    correction = torch.tensor([0.0, -1.0, 0.0, 1.0])
    many = torch.randn((40, 7), generator=torch.Generator().manual_seed(1))
    for z, c, top, scale in ((logits, correction, 2, 2.0), (logits, None, 3, 1.0), (many, 0.3 * torch.randn(7), 3, 0.5),
                             (many, torch.zeros(7), 7, 1.0)):
        tokens, experts = z.shape
        pairs = tokens * top
        ids = torch.empty(pairs, dtype=torch.int32, device="cuda")
        order, weights = torch.empty_like(ids), torch.empty(pairs, device="cuda")
        offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
        tiles = torch.empty(2 * kernels.moe_max_tiles(pairs, experts), dtype=torch.int32, device="cuda")
        count = torch.empty(1, dtype=torch.int32, device="cuda")
        kernels.moe_route(z.cuda(), top, ids, weights, offsets, order, tiles, count, all_scores="steered",
                          correction=c.cuda() if c is not None else None, weight_scale=scale)
        ids, weights = ids.view(tokens, top).cpu(), weights.view(tokens, top).cpu()
        scores = P.sigmoid(z.double().numpy())
        pick = scores + (c.double().numpy() if c is not None else 0.0)
        for t in range(tokens):
            want = P.choose(list(np.float32(pick[t])), top)
            assert ids[t].tolist() == want                  # the lower id among equals
            assert np.allclose(weights[t].numpy(), scale * scores[t][want], atol=1e-6)   # without the correction
        assert sorted(order.cpu().tolist()) == list(range(pairs))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps, norm, norm_first, weights, rot", [(1, True, False, False, 6), (1, True, True, True, 10),
                                                                 (2, True, True, True, 0), (1, False, False, False, 4),
                                                                 (2, True, False, False, 10)])
def test_heads_rotated_normed_and_laid_out(dtype, maps, norm, norm_first, weights, rot):
    from vipera_rs_amd.ops import kernels

    rng = np.random.default_rng(3)
    tokens, heads, kv_heads, dim, vdim = 9, 3, 2, 10, 14
    width = (max(maps * dim, vdim) + 15) // 16 * 16
    proj = rng.standard_normal((tokens, (heads + kv_heads) * maps * dim + kv_heads * vdim + 5))
    qw, kw = (1.0 + 0.2 * rng.standard_normal(dim), 1.0 + 0.2 * rng.standard_normal(dim)) if weights else (None, None)
    positions = rng.integers(0, 500, tokens)
    rotation = {"dims": rot, "base": 77.0}
    inv = dev(P.frequencies(rotation)) if rot else None
    qkv = torch.full((tokens, (heads * maps + 2 * kv_heads) * width), 7.0, dtype=dtype, device="cuda")
    kernels.head_prepare(dev(proj), dev(qw) if weights else None, dev(kw) if weights else None, norm, norm_first, 1e-5,
                         dev(positions, torch.int32), inv, rot, heads, kv_heads, maps, dim, vdim, width, qkv)
    got = qkv.float().cpu().numpy().reshape(tokens, heads * maps + 2 * kv_heads, width)

    def prepared(x, weight):
        if norm and norm_first:
            x = P.over_rms(x, 1e-5) * (weight if weight is not None else 1.0)
        x = P.rotate(x, positions, rotation)
        if norm and not norm_first:
            x = P.over_rms(x, 1e-5) * (weight if weight is not None else 1.0)
        return x
    q = prepared(proj[:, :heads * maps * dim].reshape(tokens, heads * maps, dim), qw)
    k = prepared(proj[:, heads * maps * dim:(heads + kv_heads) * maps * dim].reshape(tokens, kv_heads * maps, dim), kw)
    v = proj[:, (heads + kv_heads) * maps * dim:][:, :kv_heads * vdim].reshape(tokens, kv_heads, vdim)
    want = np.zeros_like(got)
    for u in range(heads * maps):
        want[:, u, (u % maps) * dim:(u % maps + 1) * dim] = q[:, u]
    want[:, heads * maps:heads * maps + kv_heads, :maps * dim] = k.reshape(tokens, kv_heads, maps * dim)
    want[:, heads * maps + kv_heads:, :vdim] = v
    assert rel_err(got, want) < (1e-5 if dtype == torch.float32 else 1e-2)
    assert np.all(got[want == 0.0] == 0.0)                  # the padding is zeros, whatever the buffer held


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_taken_out_subtracted_normed_and_gated(dtype):
    from vipera_rs_amd.ops import kernels

    rng = np.random.default_rng(4)
    tokens, heads, vdim, width = 7, 3, 10, 32
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for maps in (1, 2):
        attn = dev(rng.standard_normal((tokens, heads * maps * width)), dtype)
        a = attn.float().cpu().numpy().astype(np.float64).reshape(tokens, heads, maps, width)[..., :vdim]
        gate = rng.standard_normal((tokens, heads + 3))
        out = torch.empty((tokens, heads * vdim), dtype=dtype, device="cuda")
        if maps == 2:
            kernels.head_finish(attn, out, heads, vdim, width, 2, 0.8, unit_norm=True, eps=1e-5, factor=0.6)
            want = P.over_rms(a[:, :, 0] - 0.8 * a[:, :, 1], 1e-5) * 0.6
        else:
            kernels.head_finish(attn, out, heads, vdim, width, gate=dev(gate), gate_kind="sigmoid", gate_per_head=True)
            want = a[:, :, 0] * P.sigmoid(gate[:, :heads])[:, :, None]
        assert rel_err(out.float().cpu().numpy(), want.reshape(tokens, heads * vdim)) < tol


def test_rotation_in_place_and_a_gate_per_row():
    from vipera_rs_amd.ops import kernels

    rng = np.random.default_rng(5)
    tokens, heads, dim = 11, 3, 12
    buffer = rng.standard_normal((tokens, heads * dim + 9))
    positions = rng.integers(0, 3000, tokens)
    for rot, factor in ((12, 1.0), (8, 0.25), (0, 3.0)):
        x = dev(buffer)
        rotation = {"dims": rot, "base": 1e4}
        kernels.rotate_scale(x[:, :heads * dim], dev(positions, torch.int32), dev(P.frequencies(rotation)) if rot else None,
                             rot, heads, dim, factor)
        got = x.cpu().numpy()
        want = P.rotate(buffer[:, :heads * dim].reshape(tokens, heads, dim), positions, rotation) * factor
        assert rel_err(got[:, :heads * dim], want.reshape(tokens, -1)) < 2e-4        # angles in 32-bit
        assert np.array_equal(got[:, heads * dim:], np.float32(buffer[:, heads * dim:]))
    y, g, out = rng.standard_normal((tokens, 20)), rng.standard_normal((tokens, 1)), rng.standard_normal((tokens, 20))
    into = dev(out)
    kernels.row_gate_add(dev(y), dev(g), "sigmoid", into)
    assert rel_err(into.cpu().numpy(), out + P.sigmoid(g) * y) < 1e-6


# --- each mechanism alone, as a model of one layer -------------------------------------------------------------------
SCALING = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32}
ONE_LAYER = {
    # the sliding window with a sink: full, partial and no rotation, stretched waves, grouped heads, values wider
    # and narrower than keys, one head, widths that are no multiples of 16
    "window": L.single(L.windowed(4, 2, 16, 16, 7, rot_dims=8, base=300.0, scaling=SCALING)),
    "window_full_rotation_narrow_values": L.single(L.windowed(3, 1, 24, 8, 12), width=48),
    "window_no_rotation_odd": L.single(L.windowed(2, 2, 10, 6, 5, rot_dims=0, scale=0.4), width=50),
    "window_one_head_wide_values": L.single(L.windowed(1, 1, 8, 40, 64, rot_dims=2, scale=1.0), width=40),
    "window_wide": L.single(L.windowed(5, 5, 72, 136, 100, rot_dims=32), width=136),
    # differential attention: kept first positions beside the window, none kept, more kept than the window is long
    "two_maps": L.single(L.differential(4, 2, 8, 16, 9, keep_first=3)),
    "two_maps_nothing_kept": L.single(L.differential(2, 2, 16, 8, 6, keep_first=0, diff=0.8), width=48),
    "two_maps_more_kept_than_seen": L.single(L.differential(3, 1, 10, 14, 4, keep_first=11, diff=0.1, scale=0.5), width=50),
    "two_maps_wide": L.single(L.differential(2, 1, 72, 40, 150, keep_first=70), width=72),
    # chunks with a bias by distance beside retention: at every register layout of the recurrence's kernel
    "pair": L.single(L.parallel(L.chunked(4, 2, 16, 16, 10), L.retention(2, 16, 16))),
    "pair_odd": L.single(L.parallel(L.chunked(3, 3, 10, 14, 7, bias_rows=6, bias_max=5, scale=0.4),
                                    L.retention(3, 10, 14, rot_dims=4), 1.0, 1.0), width=50),
    "pair_one_head_two_rows": L.single(L.parallel(L.chunked(1, 1, 24, 8, 33, bias_rows=2, bias_max=20),
                                                  L.retention(1, 40, 20, decay=[0.999], rot_dims=0), 0.3, 2.0), width=40),
    "pair_wide": L.single(L.parallel(L.chunked(2, 1, 72, 40, 120, bias_rows=32, bias_max=100),
                                     L.retention(2, 72, 5, base=1e6)), width=72),
    # feed-forwards beside a small mixer
    "dense": L.single(L.windowed(1, 1, 8, 8, 6), L.dense(56), width=48),
    "experts": L.single(L.windowed(1, 1, 8, 8, 6), L.moe(8, 3, 40, shared=24), width=48),
    "experts_no_shared_top_one": L.single(L.windowed(1, 1, 8, 8, 6), L.moe(5, 1, 18, scale=1.0), width=50),
    "experts_all_chosen": L.single(L.windowed(1, 1, 8, 8, 6), L.moe(3, 3, 24, scale=0.5, shared=8), width=48),
    "experts_wide": L.single(L.windowed(1, 1, 8, 8, 6), L.moe(8, 2, 160, shared=136), width=136),
}
LONG = {"experts_wide", "window_wide", "two_maps_wide", "pair_wide"}    # a prompt of 330 tokens: several tiles


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ONE_LAYER))
def test_a_mechanism_alone_whole_prompt_then_single_tokens(tmp_path, name, dtype):
    cfg = ONE_LAYER[name]
    folder = L.make_folder(tmp_path / name, cfg, 11)
    plain_cfg, w = L.load_folder(folder)
    first = 330 if name in LONG else 45
    requests = {0: L.clear_tokens(plain_cfg, w, first, 1), 1: L.clear_tokens(plain_cfg, w, 30, 2)}
    want = {r: P.forward(plain_cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype)
    plan = [[(0, first)], [(1, 19)]] + [[(1, 1)]] * 11
    check(replay(runner, requests, plan), want, TOL[dtype], name)
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


def test_pages_of_two_positions_take_the_general_kernel(tmp_path):
    """Pages that neither the tiled nor the split 32-bit kernel takes: the general kernel holds every mask, the sink and
    the bias too."""
    folder = L.make_folder(tmp_path / "l1", L.L1, 21)
    cfg, w = L.load_folder(folder)
    tokens = L.clear_tokens(cfg, w, 50, 3)
    runner = open_runner(folder, "float32", pages=64, page=2)
    for plan in ([[(0, 50)]], [[(0, 31)]] + [[(0, 1)]] * 19):
        check(replay(runner, {0: tokens}, plan), {0: P.forward(cfg, w, tokens)}, TOL["float32"], "pages of two")


def test_the_residual_after_every_layer(tmp_path):
    """32-bit, layer by layer: a fault shows in the layer that has it, not only in the logits."""
    for name, model in (("l1", L.L1), ("l2", L.L2)):
        folder = L.make_folder(tmp_path / name, model, 21)
        plain_cfg, w = L.load_folder(folder)
        tokens = L.tokens_of(model["vocab"], 40, 5)
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
        assert len(seen) == len(residuals) == 4
        for index, (got, ref) in enumerate(zip(seen, residuals)):
            assert rel_err(got.cpu().numpy(), ref) < 1e-5, f"{name}: after layer {index} ({model['layers'][index]['type']})"


# --- whole models through the step function ------------------------------------------------------------------------
@pytest.fixture(scope="module")
def l1(tmp_path_factory):
    folder = L.make_folder(tmp_path_factory.mktemp("l1"), L.L1, 31)
    return (folder,) + L.load_folder(folder)


@pytest.fixture(scope="module")
def l2(tmp_path_factory):
    folder = L.make_folder(tmp_path_factory.mktemp("l2"), L.L2, 32)
    return (folder,) + L.load_folder(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["l1", "l2"])
def test_token_by_token_equals_the_whole_prompt(request, which, dtype):
    folder, cfg, w = request.getfixturevalue(which)
    tokens = L.clear_tokens(cfg, w, 70, 7)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype, page=4 if which == "l2" and dtype == "float32" else 8, pages=128)
    whole = replay(runner, {0: tokens}, [[(0, 70)]])
    check(whole, want, TOL[dtype], "whole")
    single = replay(runner, {0: tokens}, [[(0, 1)]] * 70)      # long decoding from the very first token
    check(single, want, TOL[dtype], "token by token")
    if dtype == "float32":   # the two ways differ by rounding only
        assert rel_err(single[0], whole[0].astype(np.float64)) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 2, 5], [13, 1, 8], [16, 2], [64, 7]])
def test_portions_of_a_prompt(l1, sizes, dtype):
    """Portions cut inside pages (8), at their borders, inside windows (9, 11, 21) and chunks (13)."""
    folder, cfg, w = l1
    tokens = L.clear_tokens(cfg, w, 83, 9)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype)
    plan = [[(0, n)] for n in portions(83, sizes)]
    check(replay(runner, {0: tokens}, plan), want, TOL[dtype], f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["l1", "l2"])
def test_a_mixed_batch_equals_each_request_alone(request, which, dtype):
    """Up to four live requests of unequal lengths: portions of some beside single tokens of others; requests end and
    later ones take their slots and pages; the pool holds less than all requests together."""
    folder, cfg, w = request.getfixturevalue(which)
    lengths = {0: 61, 1: 9, 2: 40, 3: 1, 4: 33, 5: 26, 6: 2}
    requests = {r: L.clear_tokens(cfg, w, n, 40 + r) for r, n in lengths.items()}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    plan = [[(0, 20), (1, 2), (2, 7)], [(0, 1), (1, 7), (2, 2), (3, 1)], [(0, 17), (2, 1), (4, 30)],
            [(0, 2), (2, 30), (4, 1), (5, 5)], [(0, 1), (4, 1), (5, 2), (6, 2)], [(0, 20), (4, 1), (5, 19)]]
    runner = open_runner(folder, dtype, pages=22, page=8, slots=4)    # 176 positions for 172 tokens in all
    got = replay(runner, requests, plan)
    assert {r: v.shape[0] for r, v in got.items()} == lengths
    check(got, want, TOL[dtype], "mixed")
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_and_pages_that_are_used_again_start_clean(l1, dtype):
    """One slot and few pages: every request runs in the state row and the pages the one before it left full."""
    folder, cfg, w = l1
    runner = open_runner(folder, dtype, pages=9, page=8, slots=1)
    for r, (n, cut) in enumerate([(60, [60]), (41, [5, 2, 30, 1, 1, 1, 1]), (17, [1] * 17), (64, [33, 31])]):
        tokens = L.clear_tokens(cfg, w, n, 70 + r)
        got = replay(runner, {r: tokens}, [[(r, size)] for size in cut])
        check(got, {r: P.forward(cfg, w, tokens)}, TOL[dtype], f"request {r} in the used slot")
        assert runner.cache.slot(r) == -1 and runner.cache.free_slots() == 1


def test_state_rows_and_pages_full_of_nan_do_not_reach_a_new_request(l2):
    """A slot's row and a pool's pages may hold anything when a request takes them."""
    folder, cfg, w = l2
    runner = open_runner(folder, "float32", slots=2)
    for state in runner.storage.state:
        if state is not None:
            state.fill_(float("nan"))
    for kv in runner.storage.kv:
        if kv is not None:
            kv.k.fill_(float("nan"))
            kv.v.fill_(float("nan"))
    tokens = L.clear_tokens(cfg, w, 21, 4)
    want = {0: P.forward(cfg, w, tokens)}
    check(replay(runner, {0: tokens}, [[(0, 1)], [(0, 12)], [(0, 1)], [(0, 7)]]), want, TOL["float32"], "NaN rows")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [1, 2, 3, 5, 8, 13, 21, 34])
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    """Other sizes, head counts, layer orders, windows and constants than any other test's: whole prompts, a portion
    beside single tokens of two requests, and portions down to one token."""
    folder = L.make_folder(tmp_path / "any", L.random_config(seed), seed)
    cfg, w = L.load_folder(folder)
    requests = {0: L.clear_tokens(cfg, w, 90, seed), 1: L.clear_tokens(cfg, w, 21, seed + 1)}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype, pages=64, page=16 if seed % 2 else 8)
    for plan in ([[(0, 90)], [(1, 21)]], [[(0, 70), (1, 3)]] + [[(0, 1), (1, 1)]] * 18 + [[(0, 2)]],
                 [[(0, size)] for size in portions(90, [2, 7, 1, 19, 3])] + [[(1, 1)]] * 21):
        check(replay(runner, requests, plan), want, TOL[dtype], f"configuration {seed}")
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


# --- edges: windows, chunks, kept first positions, far keys ------------------------------------------------------------
SHARP_TOL = {"float32": 1e-4, "bfloat16": 8e-2}    # peaked attention weights amplify the rounding of queries and keys


def edge_plans(n):
    return ([[(0, n)]], [[(0, n - 25)]] + [[(0, 1)]] * 25, [[(0, size)] for size in portions(n, [2, 7, 1, 19, 3])],
            [[(0, 1)]] * n)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size", [5, 19])
def test_the_edge_of_a_window(tmp_path, size, dtype):
    """Peaked attention, so that the one key just inside the window carries weight and the one just outside would: in
    prompts, token by token and in portions that end on, before and behind the edge."""
    cfg = L.single(L.windowed(2, 1, 16, 16, size, rot_dims=8, scale=0.6), vocab=61)
    folder = L.make_folder(tmp_path / "edge", cfg, 8)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 60, 17)
    want = P.forward(cfg, w, tokens)
    for off in (-1, 1):      # the test has teeth: a window one off moves the logits clearly
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["mask"]["size"] = size + off
        moved = P.forward(other, w, tokens)
        assert sum(rel_err(moved[t], want[t]) > 1e-2 for t in range(size, 60)) > 15
    runner = open_runner(folder, dtype, pages=16, page=8)
    for plan in edge_plans(60):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], f"window of {size}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size, keep", [(5, 3), (19, 6), (8, 8)])
def test_kept_first_positions_beside_a_window(tmp_path, size, keep, dtype):
    cfg = L.single(L.differential(2, 1, 16, 16, size, keep_first=keep, scale=0.5), vocab=61)
    folder = L.make_folder(tmp_path / "keep", cfg, 8, sharp=2.0)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 70, 18)
    want = P.forward(cfg, w, tokens)
    for key, off in (("keep_first", -1), ("keep_first", 1), ("size", -1), ("size", 1)):
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["mask"][key] += off
        moved = P.forward(other, w, tokens)
        assert sum(rel_err(moved[t], want[t]) > 1e-2 for t in range(size + keep, 70)) > 15, (key, off)
    runner = open_runner(folder, dtype, pages=16, page=8)
    for plan in edge_plans(70):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], f"window of {size}, {keep} kept")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size", [5, 19])
def test_the_edge_of_a_chunk_and_the_bias_by_distance(tmp_path, size, dtype):
    """Chunks are counted from position 0 of the sequence, wherever a portion starts; the right half is silenced so that
    the left one alone carries the logits."""
    cfg = L.single(L.parallel(L.chunked(2, 1, 16, 16, size, bias_rows=6, bias_max=12, scale=0.5), L.retention(1, 8, 8),
                              1.0, 0.0), vocab=61)
    folder = L.make_folder(tmp_path / "chunk", cfg, 8, sharp=2.0)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 60, 19)
    want = P.forward(cfg, w, tokens)
    for off in (-1, 1):
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["left"]["mask"]["size"] = size + off
        moved = P.forward(other, w, tokens)
        assert sum(rel_err(moved[t], want[t]) > 1e-2 for t in range(size, 60)) > 15
    flat = dict(w)
    flat["l0.mix.left.rel"] = np.zeros_like(w["l0.mix.left.rel"])
    assert sum(rel_err(P.forward(cfg, flat, tokens)[t], want[t]) > 1e-2 for t in range(60)) > 15   # the bias matters
    calm = dict(w)
    calm["l0.mix.left.sink"] = w["l0.mix.left.sink"] - 30.0
    assert sum(rel_err(P.forward(cfg, calm, tokens)[t], want[t]) > 1e-2 for t in range(60)) > 15   # and so does the sink
    runner = open_runner(folder, dtype, pages=16, page=8)
    for plan in edge_plans(60):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], f"chunks of {size}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["window", "two_maps", "chunk"])
def test_a_far_key_among_hundreds(tmp_path, kind, dtype):
    """Peaked attention over 400 positions with a window or a chunk of 256: a late query puts most of its weight on
    single keys anywhere among its visible positions, hundreds of positions and many pages back; portions end on page
    borders, one before and one behind them."""
    layer = {"window": L.windowed(2, 1, 16, 24, 256, rot_dims=8, scale=0.6),
             "two_maps": L.differential(2, 1, 16, 24, 200, keep_first=40, scale=0.5),
             "chunk": L.parallel(L.chunked(2, 1, 16, 24, 256, bias_rows=16, bias_max=200, scale=0.5), L.retention(1, 8, 8),
                                 1.0, 0.0)}[kind]
    cfg = L.single(layer, vocab=61)
    folder = L.make_folder(tmp_path / "far", cfg, 8, sharp=2.0)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 400, 17)
    want = P.forward(cfg, w, tokens)
    # the test has teeth: other tokens far back (inside the window; among the kept first positions, 300 back; at the
    # start of the chunk) move the late positions' logits clearly
    first, last = {"window": (100, 150), "two_maps": (0, 40), "chunk": (256, 290)}[kind]
    cut = P.forward(cfg, w, tokens[:first] + L.tokens_of(61, last - first, 99) + tokens[last:])
    assert sum(rel_err(cut[t], want[t]) > 1e-2 for t in range(300, 400)) > 30
    runner = open_runner(folder, dtype, pages=60, page=16)
    for plan in ([[(0, 400)]], [[(0, 340)]] + [[(0, 1)]] * 60, [[(0, n)] for n in portions(400, [127, 2, 64, 33])],
                 [[(0, 16)], [(0, 15)], [(0, 17)], [(0, 208)]] + [[(0, 1)]] * 12 + [[(0, 132)]]):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], f"far key, {kind}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim, vdim", [(64, 64), (128, 96)])
def test_a_long_prompt_on_the_prompt_kernels_of_full_head_widths(tmp_path, dim, vdim, dtype):
    """1,300 tokens through a window with a sink and through two maps with kept first positions at head widths that the
    matrix-core kernels take as they are."""
    cfg = L.config(61, 64, [L.windowed(4, 2, dim, vdim, 300, rot_dims=dim // 2),
                            L.differential(2, 1, dim // 2, vdim, 200, keep_first=70)], [None, None])
    folder = L.make_folder(tmp_path / "long", cfg, 12)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 1300, 23)
    want = P.forward(cfg, w, tokens)
    runner = open_runner(folder, dtype, pages=90, page=16)
    for plan in ([[(0, 1300)]], [[(0, 700)], [(0, 590)]] + [[(0, 1)]] * 10):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "long prompt")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_retention_that_forgets_slowly_remembers_the_first_tokens(tmp_path, dtype):
    """Decays near one: after 300 tokens, in pieces, the first tokens still weigh in the output, which a state that is
    lost or cleared between steps would not show.  The left half is silenced."""
    cfg = L.single(L.parallel(L.chunked(1, 1, 8, 8, 16), L.retention(2, 16, 16, decay=[0.998, 1.0], rot_dims=8), 0.0, 1.0),
                   vocab=61, width=32)
    folder = L.make_folder(tmp_path / "slow", cfg, 9)
    cfg, w = L.load_folder(folder)
    tokens = L.tokens_of(61, 300, 19)
    want = P.forward(cfg, w, tokens)
    other = P.forward(cfg, w, L.tokens_of(61, 150, 20) + tokens[150:])
    assert rel_err(other[-20:], want[-20:]) > 0.05            # the first half matters to the end
    runner = open_runner(folder, dtype)
    for plan in ([[(0, 300)]], [[(0, n)] for n in portions(300, [150, 1, 1, 2, 97])], [[(0, 260)]] + [[(0, 1)]] * 40):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "slow state")


def test_the_first_tokens_of_a_sequence(l1):
    """Positions 0 to 4 one by one and as a portion: nothing before position 0 exists (no state, no keys but the
    token's own beside the sink)."""
    folder, cfg, w = l1
    runner = open_runner(folder, "float32")
    for n in (1, 2, 3, 5):
        tokens = L.tokens_of(cfg["vocab"], n, 90 + n)
        want = {0: P.forward(cfg, w, tokens)}
        check(replay(runner, {0: tokens}, [[(0, n)]]), want, TOL["float32"], f"{n} tokens at once")
        check(replay(runner, {0: tokens}, [[(0, 1)]] * n), want, TOL["float32"], f"{n} tokens one by one")


# --- the engine: scheduler, sampling, captured steps ------------------------------------------------------------------
@pytest.mark.parametrize("dtype, graphs, pipelined", [("float32", False, False), ("float32", True, False),
                                                      ("float32", True, True), ("bfloat16", True, True)])
def test_greedy_generation_through_the_engine(l1, dtype, graphs, pipelined):
    from vipera_rs_amd import Engine

    folder, cfg, w = l1
    prompts = [L.tokens_of(cfg["vocab"], n, 60 + n) for n in (5, 37, 18, 2, 23)]
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


def test_the_command_line_generates(l2):
    """``bin/vipera generate`` on a Lurirax folder: the model is found by its configuration and run through the engine."""
    folder, cfg, w = l2
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = L.tokens_of(cfg["vocab"], 11, 3)
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "vipera"), "generate", folder, "--prompt-ids",
                           " ".join(str(t) for t in prompt), "--max-tokens", "8", "--dtype", "float32", "--json"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    report = json.loads(done.stdout)
    assert report["prompt_tokens"] == 11 and report["generated_tokens"] == 8
    logits = P.forward(cfg, w, prompt + report["tokens"][:-1])
    assert assert_tokens_follow_plain(logits, len(prompt), report["tokens"], 2.5e-5, "command line") >= 4


def test_the_trace_runner_replays_a_schedule(tmp_path, l1):
    """``bin/trace_run`` on a Lurirax folder: four slots, pages for the live requests only."""
    folder, cfg, w = l1
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = L.tokens_of(cfg["vocab"], 50, 1), L.tokens_of(cfg["vocab"], 20, 2)
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
