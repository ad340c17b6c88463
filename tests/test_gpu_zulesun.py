"""Zulesun on the GPU against the plain implementation (``plain/zulesun_plain.py``): kernels and mechanisms alone, then
whole models through the step function (whole prompts, single tokens, portions down to two tokens, mixed batches,
slots and pages that are used again, the edges of blocks of positions, far keys), and greedy generation through the
engine.

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

import zulesun_helpers as Z
from helpers import assert_tokens_follow_plain, rel_err
from plain import zulesun_plain as P

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 0.1}     # of a position's largest logit; observed 5e-5 and 0.06


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
    twenty may be over, which a fault of a block's edge, a page or a slot (whole runs of positions) still exceeds."""
    strict = tol < 1e-3
    over, total = [], 0
    for r in got:
        n = got[r].shape[0]
        for t in range(n):
            err = rel_err(got[r][t], want[r][t])
            total += 1
            if not err < tol:
                assert not strict, f"{label}: request {r}, position {t} of {n}: relative error {err:.3g}"
                over.append((r, t, round(err, 3)))
    assert len(over) <= total // 20, f"{label}: {len(over)} of {total} positions are over {tol}: {over[:8]}"


def tokens_for(cfg, w, count, seed):
    return Z.clear_tokens(cfg, w, count, seed)


def portions(total, sizes):
    out, k = [], 0
    while total:
        size = min(sizes[k % len(sizes)], total)
        out.append(size)
        total -= size
        k += 1
    return out


# --- kernels alone ------------------------------------------------------------------------------------------------
def route_on_device(logits, top, **how):
    from vipera_rs_amd.ops import kernels

    tokens, experts = logits.shape
    pairs = tokens * top
    ids = torch.empty(pairs, dtype=torch.int32, device="cuda")
    order, weights = torch.empty_like(ids), torch.empty(pairs, device="cuda")
    offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
    tiles = torch.empty(2 * kernels.moe_max_tiles(pairs, experts), dtype=torch.int32, device="cuda")
    count = torch.empty(1, dtype=torch.int32, device="cuda")
    kernels.moe_route(logits.cuda(), top, ids, weights, offsets, order, tiles, count, **how)
    return ids.view(tokens, top).cpu(), weights.view(tokens, top).cpu(), offsets.cpu(), order.cpu()


def test_routing_within_the_best_groups_weighs_by_the_softmax_over_all_experts():
    logits = torch.tensor([[0.5, 2.0, 1.9, -1.0, 1.8, 0.0, 0.25, 1.7],       # groups of two: (0,1) (2,3) (4,5) (6,7)
                           [3.0, -3.0, 0.0, 0.0, 0.0, 0.0, 1.0, 1.0],        # equal groups: the lower one wins
                           [-5.0, -5.0, -5.0, -5.0, -5.0, -5.0, -5.0, -5.0]])
    ids, weights, offsets, order = route_on_device(logits, 3, groups=4, keep=2, all_scores=True)
    assert ids.tolist() == [[1, 2, 0], [0, 6, 7], [0, 1, 2]]
    scores = torch.softmax(logits, dim=1)
    assert torch.allclose(weights, torch.gather(scores, 1, ids.long()), atol=1e-7)
    assert float(weights[0].sum()) < 0.9        # not renormalized
    # every group kept: the plain top-3; the weights still come from all eight
    ids, weights, _, _ = route_on_device(logits, 3, groups=4, keep=4, all_scores=True)
    assert ids.tolist() == [[1, 2, 4], [0, 6, 7], [0, 1, 2]]
    assert torch.allclose(weights, torch.gather(scores, 1, ids.long()), atol=1e-7)
    # one group kept of two halves, and the weights over the chosen only
    ids, weights, offsets, order = route_on_device(logits, 2, groups=2, keep=1)
    assert ids.tolist() == [[1, 2], [0, 2], [0, 1]]
    assert torch.allclose(weights.sum(dim=1), torch.ones(3), atol=1e-6)
    sizes = np.diff(offsets.numpy())
    assert sizes.tolist() == [2, 2, 2, 0, 0, 0, 0, 0] and sorted(order.tolist()) == list(range(6))
    # many tokens take the kernel with a wave per token
    many = torch.randn((40, 12), generator=torch.Generator().manual_seed(1))
    ids, weights, _, _ = route_on_device(many, 2, groups=3, keep=1, all_scores=True)
    full = torch.softmax(many.double(), dim=1).numpy()
    for t in range(40):
        want = P.route(full[t], 2, 3, 1)
        assert ids[t].tolist() == want and np.allclose(weights[t].numpy(), full[t][want], atol=1e-6)


@pytest.mark.parametrize("sizes", [(2, 10, 14), (3, 24, 8), (1, 40, 20), (2, 72, 5), (1, 136, 33)])
def test_the_decay_rule_alone(sizes):
    """All register layouts of the recurrence (one to sixteen key channels a lane), in pieces with the state between."""
    from vipera_rs_amd.ops import kernels

    heads, dim, vdim = sizes
    rng = np.random.default_rng(5)
    tokens = 37
    q, k = rng.standard_normal((tokens, heads * dim)), rng.standard_normal((tokens, heads * dim))
    v = rng.standard_normal((tokens, heads * vdim))
    decay = np.linspace(0.6, 0.99, heads)
    want = np.zeros((tokens, heads, vdim))
    for h in range(heads):
        state = np.zeros((dim, vdim))
        for t in range(tokens):
            state = decay[h] * state + np.outer(P.silu(k[t, h * dim:(h + 1) * dim]), P.silu(v[t, h * vdim:(h + 1) * vdim]))
            want[t, h] = state.T @ P.silu(q[t, h * dim:(h + 1) * dim])
    dev = lambda a, dt=torch.float32: torch.tensor(np.asarray(a), dtype=dt, device="cuda")
    proj = dev(np.concatenate([q, k, v], axis=1))
    floats = heads * kernels.decay_rule_head_floats(dim, vdim)
    state = torch.full((3, floats + 5), float("nan"), device="cuda")       # a row that was never cleared
    out = torch.empty((tokens, heads * vdim), device="cuda")
    at = 0
    for size in (20, 1, 2, 14):      # one entry at a time, in slot 1
        piece = slice(at, at + size)
        kernels.decay_rule(proj[piece, :heads * dim], proj[piece, heads * dim:2 * heads * dim], proj[piece, 2 * heads * dim:],
                           True, dev(decay), state, dev([0, size], torch.int32), dev([at], torch.int32), dev([1], torch.int32),
                           heads, dim, vdim, out[piece], 1)
        at += size
    assert rel_err(out.cpu().numpy(), want.reshape(tokens, -1)) < 2e-6
    assert bool(torch.isnan(state[0]).all()) and bool(torch.isnan(state[2]).all()) and bool(torch.isnan(state[1, floats:]).all())


@pytest.mark.parametrize("sizes", [(18, 5, 1), (40, 12, 3), (24, 16, 4), (7, 33, 2), (20, 100, 2), (4, 200, 5)])
def test_the_convolution_and_the_selective_scan_alone(sizes):
    """Two entries side by side in one launch, one of them continued from its state."""
    from vipera_rs_amd.ops import kernels

    channels, states, taps = sizes
    rng = np.random.default_rng(6)
    lengths = (23, 9)
    dev = lambda a, dt=torch.float32: torch.tensor(np.asarray(a), dtype=dt, device="cuda")
    conv, bias = rng.standard_normal((channels, taps)) * 0.6, rng.standard_normal(channels) * 0.2
    a_log, skip = rng.uniform(-1.5, 1.0, (channels, states)), rng.standard_normal(channels)
    dt_bias = rng.uniform(-2.0, 0.0, channels)
    streams, want = {}, {}
    for r, n in enumerate(lengths):
        s = {name: rng.standard_normal((n, width)) for name, width in
             (("x", channels), ("z", channels), ("dt", channels), ("b", states), ("c", states))}
        padded = np.concatenate([np.zeros((taps - 1, channels)), s["x"]])
        x = P.silu(sum(padded[j:j + n] * conv[:, j] for j in range(taps)) + bias)
        step = P.softplus(s["dt"] + dt_bias)
        state, y = np.zeros((channels, states)), np.zeros((n, channels))
        for t in range(n):
            state = np.exp(step[t][:, None] * -np.exp(a_log)) * state + (step[t] * x[t])[:, None] * s["b"][t][None, :]
            y[t] = state @ s["c"][t] + skip * x[t]
        streams[r], want[r] = s, y * P.silu(s["z"])
    matrices = channels * kernels.selective_scan_channel_floats(states)
    state = torch.full((3, matrices + (taps - 1) * channels), float("nan"), device="cuda")
    got = {r: [] for r in streams}
    for cut in ((15, 9), (8, 0)):       # the second request ends after the first step
        rows = [(r, streams[r], cut[r]) for r in streams if cut[r]]
        first = {0: 0, 1: 0} if cut == (15, 9) else {0: 15}
        cat = lambda name: dev(np.concatenate([s[name][first[r]:first[r] + n] for r, s, n in rows]))
        total = sum(n for _, _, n in rows)
        starts = np.cumsum([0] + [n for _, _, n in rows])
        entry_of = dev(np.repeat(np.arange(len(rows)), [n for _, _, n in rows]), torch.int32)
        meta = (dev(starts, torch.int32), dev([first[r] for r, _, _ in rows], torch.int32), dev([2 - r for r, _, _ in rows], torch.int32))
        x32 = torch.empty((total, channels), device="cuda")
        kernels.causal_conv(cat("x"), dev(conv), dev(bias), state, matrices, entry_of, *meta, x32, None, len(rows))
        out = torch.empty((total, channels), device="cuda")
        kernels.selective_scan(x32, cat("dt"), dev(dt_bias), cat("b"), cat("c"), dev(a_log), dev(skip), cat("z"), state, *meta,
                               out, len(rows))
        for (r, _, n), lo in zip(rows, starts):
            got[r].append(out[lo:lo + n].cpu().numpy())
    for r in streams:
        assert rel_err(np.concatenate(got[r]), want[r]) < 4e-6, f"request {r}"
    assert bool(torch.isnan(state[0]).all())


# --- each mechanism alone: models of one layer ---------------------------------------------------------------------
def only_left(part):
    return Z.parallel(part, Z.right(16, 4, 2, 2), 1.0, 0.0)


def only_right(part):
    return Z.parallel(Z.left(1, 1, 8, 8), part, 0.0, 1.0)


ONE_LAYER = {
    "lightning": Z.single(Z.lightning(3, 16, 24)),
    "lightning_one_head_wide_keys": Z.single(Z.lightning(1, 136, 40, [0.9]), width=40),
    "lightning_no_decay_and_none_kept": Z.single(Z.lightning(2, 8, 8, [1.0, 0.0])),
    "attention_blocks": Z.single(only_left(Z.left(4, 2, 16, 16, mask=11, softcap=3.0))),
    "attention_all_positions_partial_scaled_rotation": Z.single(only_left(Z.left(2, 1, 16, 8, rot_dims=6, base=500.0, factor=8.0))),
    "attention_values_wider_than_keys_no_rotation": Z.single(only_left(Z.left(3, 3, 8, 40, mask=16, rot_dims=0)), width=40),
    "attention_odd_widths": Z.single(only_left(Z.left(3, 1, 10, 14, mask=9, rot_dims=6, softcap=1.5)), width=50),
    "attention_many_heads": Z.single(only_left(Z.left(20, 1, 8, 8, mask=23)), width=40),      # more than one block of query heads
    "attention_wide": Z.single(only_left(Z.left(5, 5, 72, 136, mask=150, rot_dims=32)), width=136),
    "scan": Z.single(only_right(Z.right(40, 12, 5, 3))),
    "scan_one_tap_many_states": Z.single(only_right(Z.right(20, 100, 3, 1)), width=40),
    "scan_long_convolution": Z.single(only_right(Z.right(136, 16, 8, 7)), width=72),
    "both_sides": Z.single(Z.parallel(Z.left(2, 2, 16, 16, mask=8), Z.right(24, 8, 4, 4), 1.2, 0.8)),
    "dense": Z.single(Z.lightning(1, 8, 8), Z.dense(56), width=48),
    "experts": Z.single(Z.lightning(1, 8, 8), Z.moe(8, 3, 40, groups=4, keep=2), width=48),
    "experts_all_chosen": Z.single(Z.lightning(1, 8, 8), Z.moe(3, 3, 24), width=48),
    "experts_wide_one_group_of_four": Z.single(Z.lightning(1, 8, 8), Z.moe(8, 2, 160, groups=4, keep=1), width=136),
    "side_table": Z.single(Z.lightning(1, 8, 8), None, width=48, side=5),
}
LONG = {"experts_wide_one_group_of_four", "attention_wide"}       # a prompt of 330 tokens: several tiles per expert and per head


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ONE_LAYER))
def test_a_mechanism_alone_whole_prompt_then_single_tokens(tmp_path, name, dtype):
    cfg = ONE_LAYER[name]
    folder = Z.make_folder(tmp_path / name, cfg, 11)
    plain_cfg, w = Z.load_folder(folder)
    first = 330 if name in LONG else 45
    requests = {0: tokens_for(plain_cfg, w, first, 1), 1: tokens_for(plain_cfg, w, 30, 2)}
    want = {r: P.forward(plain_cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype)
    plan = [[(0, first)], [(1, 19)]] + [[(1, 1)]] * 11
    check(replay(runner, requests, plan), want, TOL[dtype], name)
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


def test_the_residual_after_every_layer(tmp_path):
    """32-bit, layer by layer: a fault shows in the layer that has it, not only in the logits."""
    folder = Z.make_folder(tmp_path / "z1", Z.Z1, 21)
    plain_cfg, w = Z.load_folder(folder)
    tokens = Z.tokens_of(Z.Z1["vocab"], 40, 5)
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
        assert rel_err(got.cpu().numpy(), ref) < 1e-5, f"after layer {index} ({Z.Z1['layers'][index]['type']})"


# --- whole models through the step function ------------------------------------------------------------------------
@pytest.fixture(scope="module")
def z1(tmp_path_factory):
    folder = Z.make_folder(tmp_path_factory.mktemp("z1"), Z.Z1, 31)
    return (folder,) + Z.load_folder(folder)


@pytest.fixture(scope="module")
def z2(tmp_path_factory):
    folder = Z.make_folder(tmp_path_factory.mktemp("z2"), Z.Z2, 32)
    return (folder,) + Z.load_folder(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["z1", "z2"])
def test_token_by_token_equals_the_whole_prompt(request, which, dtype):
    folder, cfg, w = request.getfixturevalue(which)
    tokens = tokens_for(cfg, w, 70, 7)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype, page=4 if which == "z2" else 8, pages=128 if which == "z2" else 64)
    whole = replay(runner, {0: tokens}, [[(0, 70)]])
    check(whole, want, TOL[dtype], "whole")
    single = replay(runner, {0: tokens}, [[(0, 1)]] * 70)      # long decoding from the very first token
    check(single, want, TOL[dtype], "token by token")
    if dtype == "float32":   # the two ways differ by rounding only
        assert rel_err(single[0], whole[0].astype(np.float64)) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 2, 5], [13, 1, 8], [29, 2], [64, 7]])
def test_portions_of_a_prompt(z1, sizes, dtype):
    """Portions cut inside pages (8), inside both kinds of blocks (13, 29) and inside the convolutions' reach (3, 4 taps)."""
    folder, cfg, w = z1
    tokens = tokens_for(cfg, w, 83, 9)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype)
    plan = [[(0, n)] for n in portions(83, sizes)]
    check(replay(runner, {0: tokens}, plan), want, TOL[dtype], f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["z1", "z2"])
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
def test_a_slot_and_pages_that_are_used_again_start_clean(z1, dtype):
    """One slot and few pages: every request runs in the state row and the pages the one before it left full."""
    folder, cfg, w = z1
    runner = open_runner(folder, dtype, pages=9, page=8, slots=1)
    for r, (n, cut) in enumerate([(60, [60]), (41, [5, 2, 30, 1, 1, 1, 1]), (17, [1] * 17), (64, [33, 31])]):
        tokens = tokens_for(cfg, w, n, 70 + r)
        got = replay(runner, {r: tokens}, [[(r, size)] for size in cut])
        check(got, {r: P.forward(cfg, w, tokens)}, TOL[dtype], f"request {r} in the used slot")
        assert runner.cache.slot(r) == -1 and runner.cache.free_slots() == 1


def test_a_model_without_attention_keeps_no_pages(tmp_path):
    cfg = Z.config(61, 32, [Z.lightning(2, 8, 8), Z.lightning(1, 16, 8)], [Z.dense(24), None], side=3)
    folder = Z.make_folder(tmp_path / "flat", cfg, 4)
    cfg, w = Z.load_folder(folder)
    requests = {0: Z.tokens_of(61, 50, 1), 1: Z.tokens_of(61, 12, 2)}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, "float32", pages=2, slots=2)
    plan = [[(0, 30), (1, 2)], [(0, 1), (1, 9)], [(0, 19), (1, 1)]]
    check(replay(runner, requests, plan), want, TOL["float32"], "no attention")


# --- the edges of blocks of positions, and far keys -------------------------------------------------------------------
SHARP_TOL = {"float32": 1e-4, "bfloat16": 8e-2}    # peaked attention weights amplify the rounding of queries and keys


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("size", [5, 19])
def test_the_edge_of_a_block_in_prompts_and_in_decoding(tmp_path, size, dtype):
    """Nearly even attention weights: every visible key carries about one share of a token's output, so blocks that
    are one position off, or counted from where a portion starts, move most tokens."""
    cfg = Z.single(only_left(Z.left(2, 1, 16, 16, mask=size, scale=0.05)), vocab=61)
    folder = Z.make_folder(tmp_path / "edge", cfg, 3)
    cfg, w = Z.load_folder(folder)
    tokens = Z.tokens_of(cfg["vocab"], 90, 13)
    want = P.forward(cfg, w, tokens)
    if dtype == "float32" or size == 5:      # the test has teeth
        for other in (size - 1, size + 1):
            moved = json.loads(json.dumps(cfg))
            moved["layers"][0]["mixer"]["left"]["mask"]["size"] = other
            shifted = P.forward(moved, w, tokens)
            far_off = sum(rel_err(shifted[t], want[t]) > 2 * TOL[dtype] for t in range(size, 90))
            assert far_off > 40, f"blocks of {other} move only {far_off} positions clearly"
    runner = open_runner(folder, dtype, pages=12, page=8)
    for plan in ([[(0, 90)]], [[(0, 40)]] + [[(0, 1)]] * 50, [[(0, n)] for n in portions(90, [size, 2, size + 1, 7])],
                 [[(0, size - 1)], [(0, 2)], [(0, size - 1)], [(0, 90 - 2 * size)]]):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "block edge")
    assert runner.cache.check() == ""


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mask", [0, 256])
def test_a_far_key_among_hundreds(tmp_path, mask, dtype):
    """Peaked attention (the norms' weights scaled up, a high cap): a late query puts most of its weight on single keys
    anywhere among its visible positions, hundreds of positions and many pages back, so a key that is lost or
    misplaced shows; with blocks of 256 the keys just before a block's first position must not be seen."""
    cfg = Z.single(only_left(Z.left(2, 1, 16, 16, mask=mask, rot_dims=8, scale=0.25, softcap=30.0)), vocab=61)
    folder = Z.make_folder(tmp_path / "far", cfg, 8, sharp=2.0)
    cfg, w = Z.load_folder(folder)
    tokens = Z.tokens_of(cfg["vocab"], 400, 17)
    want = P.forward(cfg, w, tokens)
    if mask:
        open_cfg = json.loads(json.dumps(cfg))
        del open_cfg["layers"][0]["mixer"]["left"]["mask"]
        unmasked = P.forward(open_cfg, w, tokens)
        assert sum(rel_err(unmasked[t], want[t]) > 0.2 for t in range(256, 400)) > 70     # the mask matters
    runner = open_runner(folder, dtype, pages=60, page=16)
    for plan in ([[(0, 400)]], [[(0, 340)]] + [[(0, 1)]] * 60, [[(0, n)] for n in portions(400, [127, 2, 64, 33])],
                 [[(0, 250)]] + [[(0, 1)]] * 12 + [[(0, 138)]]):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], "far key")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim, mask", [(64, 300), (128, 0)])
def test_a_long_prompt_on_the_prompt_kernels_of_full_head_widths(tmp_path, dim, mask, dtype):
    """Head widths of 64 and 128 take the prompt kernels that load tiles straight into LDS, which for a long prompt of
    few heads cut a tile's positions into chunks or halves: blocks of 300 positions, capped scores and all positions
    must come out of them as out of the others."""
    cfg = Z.single(only_left(Z.left(4, 2, dim, dim, mask=mask, rot_dims=dim // 2, factor=4.0, softcap=10.0)), vocab=61, width=64)
    folder = Z.make_folder(tmp_path / "long", cfg, 12)
    cfg, w = Z.load_folder(folder)
    tokens = Z.tokens_of(cfg["vocab"], 1300, 23)
    want = P.forward(cfg, w, tokens)
    runner = open_runner(folder, dtype, pages=90, page=16)
    for plan in ([[(0, 1300)]], [[(0, 700)], [(0, 590)]] + [[(0, 1)]] * 10):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "long prompt")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slow_head_remembers_the_first_tokens(tmp_path, dtype):
    """A head that forgets nothing beside one that forgets at once: after 300 tokens, in pieces, the first tokens still
    weigh as much as the last, which a state that is lost or cleared between steps would not show."""
    cfg = Z.single(Z.lightning(2, 16, 16, [1.0, 0.3]), vocab=61, width=32)
    folder = Z.make_folder(tmp_path / "slow", cfg, 9)
    cfg, w = Z.load_folder(folder)
    tokens = Z.tokens_of(cfg["vocab"], 300, 19)
    want = P.forward(cfg, w, tokens)
    forgot = P.forward(cfg, w, tokens[150:])
    assert rel_err(forgot[-20:], want[-20:]) > 0.05            # the first half matters to the end
    runner = open_runner(folder, dtype)
    for plan in ([[(0, 300)]], [[(0, n)] for n in portions(300, [150, 1, 1, 2, 97])], [[(0, 260)]] + [[(0, 1)]] * 40):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "slow head")


def test_the_first_tokens_of_a_sequence(z1):
    """Positions 0 to 4 one by one and as a portion: nothing before position 0 exists (no state, zeros before the
    convolution's start, a block that starts at the sequence's start)."""
    folder, cfg, w = z1
    runner = open_runner(folder, "float32")
    for n in (1, 2, 3, 5):
        tokens = Z.tokens_of(cfg["vocab"], n, 90 + n)
        want = {0: P.forward(cfg, w, tokens)}
        check(replay(runner, {0: tokens}, [[(0, n)]]), want, TOL["float32"], f"{n} tokens at once")
        check(replay(runner, {0: tokens}, [[(0, 1)]] * n), want, TOL["float32"], f"{n} tokens one by one")


# --- the engine: scheduler, sampling, captured steps ------------------------------------------------------------------
@pytest.mark.parametrize("dtype, graphs, pipelined", [("float32", False, False), ("float32", True, False),
                                                      ("float32", True, True), ("bfloat16", True, True)])
def test_greedy_generation_through_the_engine(z1, dtype, graphs, pipelined):
    from vipera_rs_amd import Engine

    folder, cfg, w = z1
    prompts = [Z.tokens_of(cfg["vocab"], n, 60 + n) for n in (5, 37, 18, 2, 23)]
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


def test_the_command_line_generates(z2):
    """``bin/vipera generate`` on a Zulesun folder: the model is found by its configuration and run through the engine."""
    folder, cfg, w = z2
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = Z.tokens_of(cfg["vocab"], 11, 3)
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "vipera"), "generate", folder, "--prompt-ids",
                           " ".join(str(t) for t in prompt), "--max-tokens", "8", "--dtype", "float32", "--json"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    report = json.loads(done.stdout)
    assert report["prompt_tokens"] == 11 and report["generated_tokens"] == 8
    logits = P.forward(cfg, w, prompt + report["tokens"][:-1])
    assert assert_tokens_follow_plain(logits, len(prompt), report["tokens"], 2.5e-5, "command line") >= 4


def test_the_trace_runner_replays_a_schedule(tmp_path, z1):
    """``bin/trace_run`` on a Zulesun folder: four slots, pages for the live requests only."""
    folder, cfg, w = z1
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = Z.tokens_of(cfg["vocab"], 50, 1), Z.tokens_of(cfg["vocab"], 20, 2)
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
