"""Gilidra on the GPU against the plain implementation (``plain/gilidra_plain.py``): each mechanism alone, then
whole models through the step function (whole prompts, single tokens, portions down to two tokens, mixed batches,
slots and pages that are used again, windows' edges, far keys), and greedy generation through the engine.

The plain implementation runs whole sequences in float64; every check feeds the engine's logits at all positions
of a request, however they were cut into steps, against its logits of the whole sequence.
"""
import numpy as np
import pytest
import torch

import gilidra_helpers as G
from helpers import assert_tokens_follow_plain, rel_err
from plain import gilidra_plain as P

pytestmark = pytest.mark.gpu

TOL = {"float32": 4e-5, "bfloat16": 0.1}


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
    logits (and, through the recurrent layers' state, a few after it) by more than rounding: there one position
    in twenty may be over, which a fault of a window, a page or a slot (whole runs of positions) still exceeds."""
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


def portions(total, sizes):
    """Cut ``total`` tokens into portions that cycle through ``sizes``."""
    out, k = [], 0
    while total:
        size = min(sizes[k % len(sizes)], total)
        out.append(size)
        total -= size
        k += 1
    return out


# --- kernels alone ------------------------------------------------------------------------------------------------
def test_routing_takes_the_lowest_id_among_equal_logits_and_weighs_only_the_chosen():
    from vipera_rs_amd.ops import kernels

    logits = torch.tensor([[0.5, 2.0, 2.0, -1.0, 2.0, 0.0, 0.25],
                           [3.0, -3.0, 0.0, 0.0, 0.0, 0.0, 1.0],
                           [-5.0, -5.0, -5.0, -5.0, -5.0, -5.0, -5.0]], device="cuda")
    tokens, experts, top = 3, 7, 3
    pairs = tokens * top
    ids = torch.empty(pairs, dtype=torch.int32, device="cuda")
    order, weights = torch.empty_like(ids), torch.empty(pairs, device="cuda")
    offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
    tiles = torch.empty(2 * kernels.moe_max_tiles(pairs, experts), dtype=torch.int32, device="cuda")
    count = torch.empty(1, dtype=torch.int32, device="cuda")
    kernels.moe_route(logits, top, ids, weights, offsets, order, tiles, count)
    assert ids.view(tokens, top).tolist() == [[1, 2, 4], [0, 6, 2], [0, 1, 2]]
    want = torch.softmax(torch.tensor([[2.0, 2.0, 2.0], [3.0, 1.0, 0.0], [-5.0, -5.0, -5.0]]), dim=1)
    assert torch.allclose(weights.view(tokens, top).cpu(), want, atol=1e-6)
    sizes = np.diff(offsets.cpu().numpy())
    assert sizes.tolist() == [2, 2, 3, 0, 1, 0, 1] and int(count) == 5
    placed = order.cpu().numpy()
    assert sorted(placed.tolist()) == list(range(pairs))
    chosen = ids.cpu().numpy()
    for e in range(experts):   # every place of an expert's run holds a pair that chose it
        assert all(chosen[p] == e for p in placed[offsets[e]:offsets[e + 1]])


@pytest.mark.parametrize("sizes", [(37, 3, 20, 70, 28, 75), (150, 2, 72, 140, 80, 144), (5, 3, 136, 24, 136, 24)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_product_per_head_reads_and_writes_strided_heads(dtype, sizes):
    """The second and third sizes run on the matrix cores in bfloat16 (K and the strides are multiples of 8)."""
    from vipera_rs_amd.ops import kernels

    gen = torch.Generator().manual_seed(4)
    tokens, heads, k, n, a_head, out_head = sizes
    a = torch.randn((tokens, heads * a_head), generator=gen).to(dtype).cuda()
    w = (torch.randn((heads, n, k), generator=gen) / k ** 0.5).to(dtype).cuda()
    out = torch.full((tokens, heads * out_head), 7.0, dtype=dtype, device="cuda")
    kernels.head_linear(a, a_head, k, w, out, out_head)
    got = out.float().cpu().view(tokens, heads, out_head)
    want = torch.einsum("thk,hnk->thn", a.float().cpu().view(tokens, heads, a_head)[:, :, :k], w.float().cpu())
    assert rel_err(got[:, :, :n].numpy(), want.numpy().astype(np.float64)) < (1e-5 if dtype == torch.float32 else 1e-2)
    assert bool((got[:, :, n:] == 7.0).all())          # columns between the heads' outputs are left alone


# --- each mechanism alone: models of one layer ---------------------------------------------------------------------
ONE_LAYER = {
    "latent": G.single(G.latent(3, 16, 8, 24, 40, 56, window=11)),
    "latent_all_positions_partial_rotation": G.single(G.latent(2, 8, 16, 8, 24, 40, rot_dims=8, base=500.0)),
    "latent_odd_widths": G.single(G.latent(3, 10, 6, 14, 20, 30), width=48),
    "latent_one_head_no_rotation": G.single(G.latent(1, 16, 0, 16, 16, 32), width=40),
    "delta": G.single(G.delta(4, 2, 16, 24, 4)),
    "delta_one_tap_wide_values": G.single(G.delta(2, 1, 24, 80, 1)),
    "wkv": G.single(G.wkv(3, 16, 8)),
    "wkv_wide_head": G.single(G.wkv(1, 72, 4), width=40),
    "experts": G.single(G.wkv(1, 8, 4), G.moe(7, 3, 40, 0.75), width=48),
    "experts_all_chosen": G.single(G.wkv(1, 8, 4), G.moe(3, 3, 24, 2.0), width=48),
    # wider than one tile of the grouped products, one register set of the recurrences, one block of the attention
    "experts_wide": G.single(G.wkv(1, 8, 4), G.moe(4, 2, 160, 1.0), width=136),
    "delta_wide_keys": G.single(G.delta(2, 1, 96, 20, 3), width=72),
    "delta_widest_keys": G.single(G.delta(1, 1, 136, 72, 2), width=72),
    "wkv_widest_head": G.single(G.wkv(1, 136, 8), width=72),
    "latent_wide": G.single(G.latent(5, 40, 24, 72, 136, 168, window=150), width=136),
    "latent_many_heads": G.single(G.latent(20, 8, 8, 8, 16, 24, window=23), width=40),    # more than one block of query heads
}
LONG = {"experts_wide", "latent_wide"}       # these get a prompt of 330 tokens: several tiles per expert and per head


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ONE_LAYER))
def test_a_mechanism_alone_whole_prompt_then_single_tokens(tmp_path, name, dtype):
    cfg = ONE_LAYER[name]
    folder = G.make_folder(tmp_path / name, cfg, 11)
    plain_cfg, w = P.load_folder(folder)
    first = 330 if name in LONG else 45
    requests = {0: G.tokens_of(cfg["vocab"], first, 1), 1: G.tokens_of(cfg["vocab"], 30, 2)}
    want = {r: P.forward(plain_cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype)
    plan = [[(0, first)], [(1, 19)]] + [[(1, 1)]] * 11
    check(replay(runner, requests, plan), want, TOL[dtype], name)
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


def test_the_residual_after_every_layer(tmp_path):
    """32-bit, layer by layer: a fault shows in the layer that has it, not only in the logits."""
    folder = G.make_folder(tmp_path / "g1", G.G1, 21)
    plain_cfg, w = P.load_folder(folder)
    tokens = G.tokens_of(G.G1["vocab"], 40, 5)
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
        assert rel_err(got.cpu().numpy(), ref) < 1e-5, f"after layer {index} ({G.G1['layers'][index]['type']})"


# --- whole models through the step function ------------------------------------------------------------------------
@pytest.fixture(scope="module")
def g1(tmp_path_factory):
    folder = G.make_folder(tmp_path_factory.mktemp("g1"), G.G1, 31)
    return (folder,) + P.load_folder(folder)


@pytest.fixture(scope="module")
def g2(tmp_path_factory):
    folder = G.make_folder(tmp_path_factory.mktemp("g2"), G.G2, 32)
    return (folder,) + P.load_folder(folder)


# every width odd in some way: nothing is a multiple of 8, the model's width not even of 4
G3 = G.config(83, 50, [G.wkv(3, 10, 6), G.latent(3, 6, 6, 10, 14, 22, window=9), G.delta(3, 1, 10, 14, 3)],
              [G.moe(5, 2, 18, 1.0), G.moe(3, 1, 22, 1.0), G.moe(5, 2, 18, 1.0)], logit_scale=2.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_widths_that_fit_no_fast_path(tmp_path, dtype):
    folder = G.make_folder(tmp_path / "g3", G3, 41)
    cfg, w = P.load_folder(folder)
    requests = {0: G.tokens_of(cfg["vocab"], 40, 1), 1: G.tokens_of(cfg["vocab"], 21, 2)}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    runner = open_runner(folder, dtype, page=4)
    plan = [[(0, 17), (1, 2)], [(0, 2), (1, 1)], [(0, 21), (1, 1)]] + [[(1, 1)]] * 17
    check(replay(runner, requests, plan), want, TOL[dtype], "odd widths")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["g1", "g2"])
def test_token_by_token_equals_the_whole_prompt(request, which, dtype):
    folder, cfg, w = request.getfixturevalue(which)
    tokens = G.tokens_of(cfg["vocab"], 70, 7)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype)
    whole = replay(runner, {0: tokens}, [[(0, 70)]])
    check(whole, want, TOL[dtype], "whole")
    single = replay(runner, {0: tokens}, [[(0, 1)]] * 70)      # long decoding from the very first token
    check(single, want, TOL[dtype], "token by token")
    if dtype == "float32":   # the two ways differ by rounding only
        assert rel_err(single[0], whole[0].astype(np.float64)) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 2, 5], [13, 1, 8], [29, 2], [64, 7]])
def test_portions_of_a_prompt(g1, sizes, dtype):
    """Portions cut inside pages (8), inside both windows (13, 29) and inside the convolution's reach (4 taps)."""
    folder, cfg, w = g1
    tokens = G.tokens_of(cfg["vocab"], 83, 9)
    want = {0: P.forward(cfg, w, tokens)}
    runner = open_runner(folder, dtype)
    plan = [[(0, n)] for n in portions(83, sizes)]
    check(replay(runner, {0: tokens}, plan), want, TOL[dtype], f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["g1", "g2"])
def test_a_mixed_batch_equals_each_request_alone(request, which, dtype):
    """Up to four live requests of unequal lengths: portions of some beside single tokens of others; requests end
    and later ones take their slots and pages; the pool holds less than all requests together."""
    folder, cfg, w = request.getfixturevalue(which)
    lengths = {0: 61, 1: 9, 2: 40, 3: 1, 4: 33, 5: 26, 6: 2}
    requests = {r: G.tokens_of(cfg["vocab"], n, 40 + r) for r, n in lengths.items()}
    want = {r: P.forward(cfg, w, t) for r, t in requests.items()}
    plan = [[(0, 20), (1, 2), (2, 7)], [(0, 1), (1, 7), (2, 2), (3, 1)], [(0, 17), (2, 1), (4, 30)],
            [(0, 2), (2, 30), (4, 1), (5, 5)], [(0, 1), (4, 1), (5, 2), (6, 2)], [(0, 20), (4, 1), (5, 19)]]
    runner = open_runner(folder, dtype, pages=22, page=8, slots=4)    # 176 positions for 172 tokens in all
    got = replay(runner, requests, plan)
    assert {r: v.shape[0] for r, v in got.items()} == lengths
    check(got, want, TOL[dtype], "mixed")
    assert runner.cache.check() == "" and runner.cache.live_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_and_pages_that_are_used_again_start_clean(g2, dtype):
    """One slot and few pages: every request runs in the state row and the pages the one before it left full."""
    folder, cfg, w = g2
    runner = open_runner(folder, dtype, pages=9, page=8, slots=1)
    for r, (n, cut) in enumerate([(60, [60]), (41, [5, 2, 30, 1, 1, 1, 1]), (17, [1] * 17), (64, [33, 31])]):
        tokens = G.tokens_of(cfg["vocab"], n, 70 + r)
        got = replay(runner, {r: tokens}, [[(r, size)] for size in cut])
        check(got, {r: P.forward(cfg, w, tokens)}, TOL[dtype], f"request {r} in the used slot")
        assert runner.cache.slot(r) == -1 and runner.cache.free_slots() == 1


# --- windows' edges and far keys, with weights that make one key stand out -------------------------------------------
SHARP_TOL = {"float32": 4e-5, "bfloat16": 8e-2}    # peaked attention weights amplify the rounding of queries and keys


def sharp_single(window, seed, tmp_path, name):
    """One latent layer whose attention is peaked (queries and keys scaled up), so that a key that is wrongly seen
    or wrongly dropped moves the output by much more than any tolerance."""
    cfg = G.single(G.latent(2, 16, 8, 16, 32, 40, window=window, scale=1.0), vocab=61)
    folder = G.make_folder(tmp_path / name, cfg, seed, sharp=3.0)
    return (folder,) + P.load_folder(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [5, 19])
def test_the_window_edge_in_prompts_and_in_decoding(tmp_path, window, dtype):
    """Even attention weights: every visible key carries about 1 / window of a token's output, so a window that is
    one position off moves every token behind the first window (by a fifth with a window of five)."""
    cfg = G.single(G.latent(2, 16, 8, 16, 32, 40, window=window), vocab=61)
    folder = G.make_folder(tmp_path / "edge", cfg, 3)
    cfg, w = P.load_folder(folder)
    tokens = G.tokens_of(cfg["vocab"], 90, 13)
    want = P.forward(cfg, w, tokens)
    if dtype == "float32" or window == 5:      # the test has teeth
        for other in (window - 1, window + 1):
            moved = dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], mask={"size": other}))])
            shifted = P.forward(moved, w, tokens)
            far_off = sum(rel_err(shifted[t], want[t]) > 2 * TOL[dtype] for t in range(window, 90))
            assert far_off > 40, f"a window of {other} moves only {far_off} positions clearly"
    runner = open_runner(folder, dtype, pages=12, page=8)      # pages behind the window come back while the request runs
    for plan in ([[(0, 90)]], [[(0, 40)]] + [[(0, 1)]] * 50, [[(0, n)] for n in portions(90, [window, 2, window + 1, 7])]):
        check(replay(runner, {0: tokens}, plan), {0: want}, TOL[dtype], "window")
    assert runner.cache.check() == ""


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dtype):
    """No window, peaked attention: a late query puts most of its weight on single keys anywhere among 400
    positions, hundreds of positions and many pages back, so a key that is lost or misplaced shows."""
    folder, cfg, w = sharp_single(0, 8, tmp_path, "far")
    tokens = G.tokens_of(cfg["vocab"], 400, 17)
    want = P.forward(cfg, w, tokens)
    runner = open_runner(folder, dtype, pages=60, page=16)
    for plan in ([[(0, 400)]], [[(0, 340)]] + [[(0, 1)]] * 60, [[(0, n)] for n in portions(400, [127, 2, 64, 33])]):
        check(replay(runner, {0: tokens}, plan), {0: want}, SHARP_TOL[dtype], "far key")


def test_the_first_tokens_of_a_sequence(g1):
    """Positions 0 to 4 one by one and as a portion: nothing before position 0 exists (no state, zeros before the
    convolution's start, a previous token of zeros)."""
    folder, cfg, w = g1
    runner = open_runner(folder, "float32")
    for n in (1, 2, 3, 5):
        tokens = G.tokens_of(cfg["vocab"], n, 90 + n)
        want = {0: P.forward(cfg, w, tokens)}
        check(replay(runner, {0: tokens}, [[(0, n)]]), want, TOL["float32"], f"{n} tokens at once")
        check(replay(runner, {0: tokens}, [[(0, 1)]] * n), want, TOL["float32"], f"{n} tokens one by one")


# --- the engine: scheduler, sampling, captured steps ------------------------------------------------------------------
@pytest.mark.parametrize("dtype, graphs, pipelined", [("float32", False, False), ("float32", True, False),
                                                      ("float32", True, True), ("bfloat16", True, True)])
def test_greedy_generation_through_the_engine(g1, dtype, graphs, pipelined):
    from vipera_rs_amd import Engine

    folder, cfg, w = g1
    prompts = [G.tokens_of(cfg["vocab"], n, 60 + n) for n in (5, 37, 18, 2, 23)]
    new_tokens = 24
    engine = Engine(folder, dtype=dtype, block_size=8, num_blocks=40, max_num_seqs=3, chunk_size=16,
                    max_num_batched_tokens=32, max_model_len=128, use_graphs=graphs, pipelined=pipelined)
    got = engine.generate(prompts, max_new_tokens=new_tokens)
    clear = 0
    for prompt, generation in zip(prompts, got):
        assert len(generation.tokens) == new_tokens
        logits = P.forward(cfg, w, prompt + generation.tokens[:-1])
        clear += assert_tokens_follow_plain(logits, len(prompt), generation.tokens, 2.5e-5 if dtype == "float32" else 1e-2,
                                            f"{dtype}, prompt of {len(prompt)}")
    assert clear >= (100 if dtype == "float32" else 40)
    if graphs:
        assert engine.runner.graphs.replays > 0
    assert engine.runner.cache.check() == "" and engine.runner.cache.live_requests() == 0


def test_the_command_line_generates(g2):
    """``bin/vipera generate`` on a Gilidra folder: the model is found by its configuration and run through the engine."""
    import json
    import os
    import subprocess
    import sys

    folder, cfg, w = g2
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = G.tokens_of(cfg["vocab"], 11, 3)
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "vipera"), "generate", folder, "--prompt-ids",
                           " ".join(str(t) for t in prompt), "--max-tokens", "8", "--dtype", "float32", "--json"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    report = json.loads(done.stdout)
    assert report["prompt_tokens"] == 11 and report["generated_tokens"] == 8
    logits = P.forward(cfg, w, prompt + report["tokens"][:-1])
    assert assert_tokens_follow_plain(logits, len(prompt), report["tokens"], 2.5e-5, "command line") >= 4


def test_the_trace_runner_replays_a_schedule(tmp_path, g2):
    """``bin/trace_run`` on a Gilidra folder: four slots, pages for the live requests only."""
    import json
    import os
    import subprocess
    import sys

    folder, cfg, w = g2
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = G.tokens_of(cfg["vocab"], 50, 1), G.tokens_of(cfg["vocab"], 20, 2)
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
