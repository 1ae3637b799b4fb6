"""GPU: the Givizen decoder in the engine against the plain implementation (tests/plain_givizen.py): every mechanism
alone, every way of cutting and batching the same requests, reused pages and slots, keys at every edge of a window,
long decoding, other sizes, and greedy generation through the engine's own entry point."""

from __future__ import annotations

import copy
import random

import numpy as np
import pytest
import torch

import givizen_util as gu
import plain_givizen as pg
import replay_util
from conftest import random_tokens

pytestmark = pytest.mark.gpu

# a row's error: root mean square of the difference of its logits, mean taken off, as a share of the logits' own spread
LIMIT = {"float32": 2e-5, "bfloat16": 8e-2}
RMS_LIMIT = {"float32": 1e-5, "bfloat16": 3e-2}


def plain_all(raw, weights, requests):
    return {rid: pg.forward(raw, weights, tokens).float() for rid, tokens in requests.items()}


def run_and_compare(raw, weights, requests, steps, dtype, plain, page_size=16, max_running=4, limit=None, graph_decode=False):
    pool = max(replay_util.max_live_tokens(steps, page=page_size), page_size)
    runner = gu.make_runner(raw, weights, dtype, pool, page_size, max_running, graph_decode=graph_decode)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    for rid in requests:
        assert rid in rows, f"{rid}: no logits"
    worst, rms = gu.spread(rows, plain)
    assert worst <= (limit or LIMIT[dtype]) and rms <= RMS_LIMIT[dtype], (dtype, worst, rms)
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0
    return runner


ATT = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.35, "mask": {"size": 12}, "q_temp": {"coef": 0.5, "every": 6}}
MECHANISMS = {
    "attention": {"type": "attention", "mlp": None, "mixer": ATT},
    "attention_one_head_wide_values": {"type": "attention", "mlp": None,
                                       "mixer": {**ATT, "heads": 1, "kv_heads": 1, "dim": 8, "vdim": 40, "mask": {"size": 5}}},
    "attention_sees_everything": {"type": "attention", "mlp": None, "mixer": {**ATT, "mask": {"size": 4096}}},
    "attention_2": {"type": "attention_2", "mlp": None, "mixer": {**ATT, "softcap": 3.0}},
    "attention_2_many_heads_on_one": {"type": "attention_2", "mlp": None,
                                      "mixer": {**ATT, "heads": 18, "kv_heads": 1, "dim": 24, "vdim": 8, "softcap": 50.0}},
    "attention_2_window_of_one": {"type": "attention_2", "mlp": None, "mixer": {**ATT, "softcap": 2.0, "mask": {"size": 1}}},
    "experts": {"type": "attention", "mixer": {**ATT, "heads": 1, "kv_heads": 1},
                "mlp": {"kind": "moe", "router": {"experts": 7, "top": 3}, "expert": {"ff": 24, "limit": 1.0},
                        "shared": {"ff": 16, "limit": 2.0}}},
    "experts_without_shared": {"type": "attention", "mixer": {**ATT, "heads": 1, "kv_heads": 1},
                               "mlp": {"kind": "moe", "router": {"experts": 70, "top": 1}, "expert": {"ff": 8, "limit": 4.0}}},
    "experts_odd_widths": {"type": "attention", "mixer": {**ATT, "heads": 1, "kv_heads": 1},
                           "mlp": {"kind": "moe", "router": {"experts": 2, "top": 2}, "expert": {"ff": 13, "limit": 0.5},
                                   "shared": {"ff": 5, "limit": 0.25}}},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_a_mechanism_alone(name, dtype):
    """One layer of one kind: whole prompts, then the same tokens in portions down to two tokens and one by one
    (across pages, across the window's edge and the temperature's steps), three requests side by side."""
    raw = gu.single(copy.deepcopy(MECHANISMS[name]), cap=20.0 if "experts" in name else None)
    weights = gu.make_weights(raw, seed=3, exact_router=True)
    requests = {"a": random_tokens(45, raw["vocab"], 1), "b": random_tokens(21, raw["vocab"], 2), "c": [7]}
    plain = plain_all(raw, weights, requests)
    run_and_compare(raw, weights, requests, replay_util.whole(requests), dtype, plain)
    run_and_compare(raw, weights, requests, replay_util.portions(requests, sizes=(2, 3, 2, 17, 2, 5)), dtype, plain)
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, chunk_sizes=(2, 7, 3), decode_tail=9),
                    dtype, plain, max_running=3)


def test_routers_that_read_the_whole_stream():
    """float32, where rounding cannot turn a choice: routers with random weights on every coordinate, so that a
    token's experts depend on its context."""
    raw = gu.SMALL_A
    weights = gu.make_weights(raw, seed=8)
    requests = {"a": random_tokens(60, raw["vocab"], 11), "b": random_tokens(33, raw["vocab"], 12)}
    plain = plain_all(raw, weights, requests)
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=2, chunk_sizes=(9, 2, 30)), "float32", plain)


SCHEDULES = {
    "whole": replay_util.whole,
    "tail": lambda requests: replay_util.tail_one_by_one(requests, tail=40),
    "portions": replay_util.portions,
    "mixed": lambda requests: replay_util.mixed(requests, live=4),
}
LENGTHS = {"A": [5, 17, 33, 70, 100, 1], "B": [2, 9, 40, 64, 131]}


@pytest.fixture(scope="module")
def models():
    out = {}
    for index, (name, raw) in enumerate(gu.SMALL.items()):
        weights = gu.make_weights(raw, seed=20 + index, exact_router=True)
        requests = {f"{name}{i}": random_tokens(n, raw["vocab"], seed=50 + i) for i, n in enumerate(LENGTHS[name])}
        out[name] = (raw, weights, requests, plain_all(raw, weights, requests))
    return out


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("name", sorted(gu.SMALL))
def test_logits_do_not_depend_on_cutting_or_batching(models, name, schedule, dtype):
    """Prefill against token-by-token decoding (the tail is longer than every window but one), portions of several
    sizes, unequal requests in one batch against each alone; six requests take turns on four slots, and the pool is no
    larger than the schedule's peak."""
    raw, weights, requests, plain = models[name]
    run_and_compare(raw, weights, requests, SCHEDULES[schedule](requests), dtype, plain)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(gu.SMALL))
def test_captured_steps_give_the_same_logits(models, name, dtype):
    """Steps of single tokens replay captured graphs (and short mixed steps theirs, from the second time a shape
    comes), with uncaptured steps between the replays; every replay is checked against the plain logits."""
    raw, weights, requests, plain = models[name]
    steps = replay_util.fixed_portions(requests, portion=8, live=3, decode_tail=14)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = gu.make_runner(raw, weights, dtype, pool, 16, 4, graph_decode=True)
    assert runner.graphs is not None, "the model's parts all say that they may be captured"
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    worst, rms = gu.spread(rows, plain)
    assert runner.graph_replays >= 10 and runner.mixed_graph_replays > 0, (runner.graph_replays, runner.mixed_graph_replays)
    assert worst <= LIMIT[dtype] and rms <= RMS_LIMIT[dtype], (worst, rms)


@pytest.mark.parametrize("page_size", [4, 64])
def test_other_page_sizes(models, page_size):
    raw, weights, requests, plain = models["A"]
    for dtype in ("float32", "bfloat16"):
        run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=5), dtype, plain,
                        page_size=page_size, max_running=3)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_traces_reuse_pages_and_slots(models, dtype):
    """Random cuts (one token, two, up to a page's edge, one past it) of ten requests on three slots: every slot and
    page is handed out again, and pages that a window has passed go back to the pool while their request lives."""
    raw, weights, _, _ = models["B"]
    rng = random.Random(4)
    requests, steps = replay_util.random_trace(rng, [3, 40, 17, 1, 33, 64, 2, 18, 49, 31], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = gu.make_runner(raw, weights, dtype, pool, 16, 3)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert rows and set(rows) <= set(requests)
    worst, _ = gu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


NEEDLE, ASK, FILLERS = 1, 2, 40  # token ids: the one to be found, the one that looks for it, the first of the rest
WINDOW = 200


def planted(kind: str):
    """A single layer whose weights are changed by hand so that one score stands out: the token ASK looks, through a
    query dimension that only it has, for a key dimension that only the token NEEDLE has.  Per-head norms keep the
    direction, so after them the pair's product is near the head's size; the last head's slope is 2^-8 a token, so a
    needle at the far edge of the window still outweighs everything nearer."""
    mixer = {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 1.0, "mask": {"size": WINDOW},
             "q_temp": {"coef": 0.3, "every": 64}}
    if kind == "attention_2":
        mixer["softcap"] = 30.0
    raw = gu.single({"type": kind, "mlp": None, "mixer": mixer}, width=32, vocab=64)
    w = gu.make_weights(raw, seed=9)
    w["embed"][:, 0:2] = 0.0
    w["embed"][NEEDLE, 0] = 8.0
    w["embed"][ASK, 1] = 8.0
    for name, column in (("k", 0), ("q", 1)):
        w["l0.mix." + name][:, 0:2] = 0.0
        w["l0.mix." + name] *= 0.25
        for h in range(w["l0.mix." + name].shape[0] // 16):
            w["l0.mix." + name][h * 16, column] = 16.0
    if kind == "attention":
        w["l0.mix.q.norm"][:] = 1.0
        w["l0.mix.k.norm"][:] = 1.0
        w["l0.mix.sink"][:] = torch.tensor([-5.0, 9.0])  # nothing beside one head's keys, forty times their weight beside the other's
    w["l0.mix.o"] *= 4.0
    return raw, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_a_key_is_seen_up_to_the_windows_edge_and_not_beyond(kind, dtype):
    """The needle just inside the window and just outside it, at page borders, at the first positions and far back;
    asked for inside a prompt's portion and by a token decoded alone, by requests that share a pool whose pages go
    back as the window passes them.  A key lost or kept by one token too many moves these logits by far more than the
    tolerance (checked below on the plain implementation itself), and so does a sink that is left out."""
    raw, weights = planted(kind)
    length = 600
    # distance of the first asker (at `length`) to the needle: inside for >= length - WINDOW + 1
    places = [0, 1, length - WINDOW - 1, length - WINDOW, length - WINDOW + 1, length - WINDOW + 2, length - WINDOW + 3,
              447, 448, 449, 511, 512, 590, 599]
    requests = {}
    for place in places:
        tokens = [FILLERS + t % (raw["vocab"] - FILLERS) for t in random_tokens(length, 1000, 30 + place)]
        tokens[place] = NEEDLE
        requests[f"n{place}"] = tokens + [ASK, FILLERS, ASK]
    plain = plain_all(raw, weights, requests)
    # the test of the test: the asked rows change with the needle exactly where the window says so
    def moved(rid, row):
        blind = list(requests[rid])
        blind[blind.index(NEEDLE)] = FILLERS + 3
        other = pg.forward(raw, weights, blind).float()
        diff = other[row] - plain[rid][row]
        return float((diff - diff.mean()).pow(2).mean().sqrt() / plain[rid][row].std())
    inside, outside = f"n{length - WINDOW + 1}", f"n{length - WINDOW}"
    assert moved(inside, length) > 0.3 and moved(outside, length) < 1e-6
    assert moved(f"n{length - WINDOW + 3}", length + 2) > 0.3 and moved(f"n{length - WINDOW + 2}", length + 2) < 1e-6
    if kind == "attention":
        no_sink = dict(weights)
        no_sink["l0.mix.sink"] = torch.full((2,), -30.0)
        # (the layer's norm takes a factor that all heads share away again: the sinks differ between the heads)
        diff = pg.forward(raw, no_sink, requests["n590"]).float()[length + 1] - plain["n590"][length + 1]
        assert float((diff - diff.mean()).pow(2).mean().sqrt() / plain["n590"][length + 1].std()) > 0.05
    steps, sizes = [], (129, 2, 255, 31, 64, 3)
    waiting = list(requests.items())
    while waiting:
        pair = [waiting.pop(0) for _ in range(min(2, len(waiting)))]
        fed = {rid: 0 for rid, _ in pair}
        turn = 0
        while any(fed[rid] < len(tokens) for rid, tokens in pair):
            entries, end = [], []
            for index, (rid, tokens) in enumerate(pair):
                left = len(tokens) - fed[rid]
                if left == 0:
                    continue
                # the last token (an asker) comes alone; the asker before it inside a portion
                size = 1 if left == 1 else min(sizes[(turn + index) % len(sizes)], left - 1)
                want = [i for i in range(size) if fed[rid] + i >= length]
                entries.append({"id": rid, "tokens": tokens[fed[rid]: fed[rid] + size], "want": want})
                fed[rid] += size
                if fed[rid] == len(tokens):
                    end.append(rid)
            turn += 1
            steps.append({"step": len(steps), "entries": entries, "end": end})
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = gu.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == [length, length + 1, length + 2] for rid in requests)
    worst, _ = gu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst
    # the window's pages went back while the requests lived: the window group never held a whole prompt
    group = next(g for g in runner.cache.groups if g.spec.window == WINDOW)
    assert group.allocator.free_count == group.allocator.total_pages


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A prompt of 300 tokens, then 250 tokens decoded one by one: every window passes over decoded tokens, the
    temperature steps many times, pages are crossed and given back.  (bfloat16: what rounding costs over 550 rows
    is measured: the engine has to be closer to the yardstick, at its worst row and on average, than the plain
    implementation run in bfloat16 throughout.)"""
    raw = gu.SMALL_A
    weights = gu.make_weights(raw, seed=31, exact_router=True)
    requests = {"long": random_tokens(550, raw["vocab"], 7)}
    stepper = pg.Stepper(raw, weights)
    plain = {"long": torch.cat([stepper.feed([t]) for t in requests["long"]]).float()}
    steps = replay_util.tail_one_by_one(requests, tail=250)
    limit = None
    if dtype == "bfloat16":
        rough = pg.forward(raw, weights, requests["long"], dtype=torch.bfloat16).float().numpy()
        limit, rough_rms = gu.spread({"long": dict(enumerate(rough))}, plain)
        assert limit < 1.0
    runner = gu.make_runner(raw, weights, dtype, max(replay_util.max_live_tokens(steps, page=16), 16), 16, 1)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    worst, rms = gu.spread(rows, plain)
    assert worst <= (limit or LIMIT[dtype]) and rms <= (rough_rms if limit else RMS_LIMIT[dtype]), (dtype, worst, rms)
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0


def test_greedy_generation_through_the_engine(models):
    """The engine's own entry point and scheduler (prompts in portions, several requests at once) generate what the
    plain implementation generates."""
    from cie_amd import Engine, GenerationConfig
    from cie_amd.config import config_from_dict

    raw, weights, _, _ = models["A"]
    prompts = [random_tokens(n, raw["vocab"], 80 + n) for n in (3, 19, 42)]
    for dtype in ("float32", "bfloat16"):
        engine = Engine(config=config_from_dict(raw), seed=0, dtype=dtype, page_size=16, kv_tokens=512, max_running=3,
                        max_model_len=128, prefill_chunk=8, token_budget=24, prefix_cache_pages=0)
        engine.model.load(gu.Fixed(weights), dtype, "cuda:0")
        results = engine.generate(prompts, GenerationConfig(max_output_tokens=12))
        for prompt, result in zip(prompts, results):
            assert len(result.token_ids) == 12
            turned = replay_util.greedy_tokens_follow_plain(
                lambda tokens: pg.forward(raw, weights, tokens), prompt, result.token_ids,
                (lambda tokens: pg.forward(raw, weights, tokens, dtype=torch.bfloat16)) if dtype == "bfloat16" else None)
            assert turned <= (0 if dtype == "float32" else 3)


def test_the_trace_runner_replays_a_model_folder(tmp_path, models):
    """bin/trace_run on a folder written for it: same logits as the plain implementation."""
    import json
    import subprocess
    import sys

    from cie_amd.weights import write_tensors
    from conftest import ROOT

    raw, weights, requests, plain = models["A"]
    folder = write_tensors(tmp_path / "model", raw, {k: v.to(torch.bfloat16) for k, v in weights.items()})
    steps = replay_util.mixed(requests, live=4)
    out = tmp_path / "out"
    pool = replay_util.max_live_tokens(steps, page=64)
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", str(pool), "--max-requests", "4"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.split("\n") if line.startswith("done")] == [f"done {s['step']}" for s in steps]
    outputs = {s["step"]: np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, raw["vocab"])
               for s in steps if any(e["want"] for e in s["entries"])}
    worst, _ = gu.spread(replay_util.by_position(steps, outputs), plain)
    assert worst <= LIMIT["float32"], worst


# ---------------------------------------------------------------- kernels alone
def _paged(keys, values, page_size, dtype):
    """One sequence's keys [S, G, D] and values [S, G, V] laid into shuffled pages; (k_pool, v_pool, table)."""
    S, G, D = keys.shape
    V = values.shape[2]
    pages = -(-S // page_size)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(S))[:pages]
    k_pool = torch.zeros(pages + 3, G, page_size, D)
    v_pool = torch.zeros(pages + 3, G, V, page_size)
    for s in range(S):
        k_pool[order[s // page_size], :, s % page_size] = keys[s]
        v_pool[order[s // page_size], :, :, s % page_size] = values[s]
    table = torch.zeros(2, pages, dtype=torch.int32)
    table[1] = order.int()
    return k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda(), table.cuda()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 64, 64, 37), (8, 1, 128, 64, 100), (20, 1, 64, 128, 9), (3, 3, 128, 128, 1000)])
def test_attention_kernels_against_the_plain_scores(shape, dtype):
    """Both forms of the kernel, every shaping step on and off, a portion of 70 tokens behind 150 cached ones and a
    single token, against the plain scores and weights."""
    from cie_amd.kernels import ops

    H, G, D, V, window = shape
    g = torch.Generator().manual_seed(H)
    S, T = 220, 70
    q = torch.randn(S, H, D, generator=g).to(dtype).float() * 0.6
    k = torch.randn(S, G, D, generator=g).to(dtype).float()
    v = torch.randn(S, G, V, generator=g).to(dtype).float()
    gate = torch.randn(S, H + 3, generator=g).to(dtype).float() * 2
    sinks = torch.randn(H, generator=g) * 2
    slopes = pg.slopes(H, torch.float32)
    k_pool, v_pool, table = _paged(k, v, 16, dtype)
    pos = torch.arange(S)
    dev = lambda t, kind=torch.int32: torch.tensor(t, dtype=kind).cuda()
    for use in ({"cap": 2.5, "slopes": True, "sinks": True, "gate": False}, {"cap": None, "slopes": True, "sinks": False, "gate": True},
                {"cap": None, "slopes": False, "sinks": False, "gate": False}):
        kind = "attention" if use["sinks"] else "attention_2"
        p = {"scale": 0.2, "mask": {"size": window}, "softcap": use["cap"]}
        s = torch.einsum("thd,shd->hts", q.double(), k.double().repeat_interleave(H // G, 1)) * 0.2
        if use["cap"]:
            s = pg.soft_cap(s, use["cap"])
        distance = pos[:, None] - pos[None, :]
        if use["slopes"]:
            s = s - pg.slopes(H)[:, None, None] * distance[None]
        s = s.masked_fill(((distance < 0) | (distance >= window))[None], float("-inf"))
        a = pg.attention_weights(kind, s, sinks.double())
        want = torch.einsum("hts,shv->thv", a, v.double().repeat_interleave(H // G, 1))
        if use["gate"]:
            want = want * torch.sigmoid(gate[:, :H].double())[:, :, None]
        for first, count in ((S - T, T), (S - 1, 1), (0, 33)):
            rows = slice(first, first + count)
            common = dict(window=window, scale=0.2, softcap=use["cap"], slopes=slopes.cuda() if use["slopes"] else None,
                          sinks=sinks.cuda() if use["sinks"] else None,
                          gate=gate[rows].to(dtype).cuda() if use["gate"] else None)
            qd = q[rows].reshape(count, H * D).to(dtype).cuda().contiguous()
            got = ops.scored_attention_generic(qd, k_pool, v_pool, table, dev(list(range(first, first + count))),
                                               dev([0] * count), dev([1]), count, H, G, D, V, **common)
            tol = 2e-5 if dtype == torch.float32 else 2e-2
            assert torch.allclose(got.double().cpu().reshape(count, H, V), want[rows], atol=tol, rtol=tol), (use, first, "generic")
            if dtype == torch.bfloat16:
                group = H // G
                row_tiles = 1 if group <= 16 else 2
                per_tile = 16 * row_tiles // group
                firsts = list(range(0, count, per_tile))
                got = ops.scored_attention_mfma(qd, k_pool, v_pool, table, dev([0] * len(firsts)), dev(firsts), len(firsts),
                                                dev([1]), dev([first]), dev([count]), dev([0, count]), count, H, G, D, V,
                                                per_tile, row_tiles, **common)
                assert torch.allclose(got.double().cpu().reshape(count, H, V), want[rows], atol=tol, rtol=tol), (use, first, "mfma")
                # the same with every tile's keys in shares of 128, joined by the second kernel
                reach = min(first + count, window) + per_tile + 32
                got = ops.scored_attention_mfma(qd, k_pool, v_pool, table, dev([0] * len(firsts)), dev(firsts), len(firsts),
                                                dev([1]), dev([first]), dev([count]), dev([0, count]), count, H, G, D, V,
                                                per_tile, row_tiles, **common, n_splits=-(-reach // 128), keys_per_split=128)
                assert torch.allclose(got.double().cpu().reshape(count, H, V), want[rows], atol=tol, rtol=tol), (use, first, "shares")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_heads_are_normed_scaled_padded_and_cached(dtype):
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(0)
    H, G, d, v, D, DV, T = 3, 2, 12, 20, 16, 24, 9
    cols = H * d + G * d + G * v
    proj = torch.randn(T, cols + 5, generator=g).to(dtype)
    qw, kw = torch.rand(d, generator=g) + 0.5, torch.rand(d, generator=g) + 0.5
    positions = torch.tensor([0, 1, 2, 30, 31, 32, 33, 7, 8], dtype=torch.int32)
    seq_of = torch.tensor([0, 0, 0, 1, 1, 1, 1, 2, 2], dtype=torch.int32)
    slots = torch.tensor([2, 0, 1], dtype=torch.int32)
    table = torch.tensor([[5, 6, 7], [1, 2, 3], [0, 4, 8]], dtype=torch.int32)
    for mode in ("weight", "unit", None):
        k_pool = torch.full((9, G, 16, D), 9.0, dtype=dtype).cuda()
        v_pool = torch.full((9, G, DV, 16), 9.0, dtype=dtype).cuda()
        q = ops.heads_prepare(proj.cuda(), (0, H * d, H * d + G * d), H, G, d, v, D, DV, mode, qw.cuda(), kw.cuda(), 1e-5,
                              (0.5, 8), positions.cuda(), seq_of.cuda(), slots.cuda(), table.cuda(), k_pool, v_pool, T)
        x = proj.double()
        qs = x[:, : H * d].reshape(T, H, d)
        ks = x[:, H * d: H * d + G * d].reshape(T, G, d)
        if mode:
            qs, ks = qs / pg.rms(qs, 1e-5), ks / pg.rms(ks, 1e-5)
        if mode == "weight":
            qs, ks = qs * qw.double(), ks * kw.double()
        qs = qs * pg.query_temperature(positions.long(), {"coef": 0.5, "every": 8})[:, None, None]
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        got = q.double().cpu().reshape(T, H, D)
        assert torch.allclose(got[:, :, :d], qs, atol=tol, rtol=tol) and bool((got[:, :, d:] == 0).all())
        for t in range(T):
            page = int(table[slots[seq_of[t]], positions[t] // 16])
            at = int(positions[t]) % 16
            assert torch.allclose(k_pool[page, :, at, :d].double().cpu(), ks[t], atol=tol, rtol=tol)
            assert bool((k_pool[page, :, at, d:] == 0).all())
            want_v = x[t, H * d + G * d: cols].reshape(G, v)
            assert torch.allclose(v_pool[page, :, :v, at].double().cpu(), want_v, atol=tol) and bool((v_pool[page, :, v:, at] == 0).all())
        assert int((k_pool == 9).sum()) == k_pool.numel() - T * G * D  # nothing else is touched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(150, 8, 2, 64, 32), (7, 70, 1, 24, 40), (33, 3, 3, 50, 13), (600, 16, 4, 128, 64),
                                   (500, 6, 3, 328, 200)])  # (the last: several slices of k in the tiled form, and a rest)
def test_routed_experts_kernels(sizes, dtype):
    """Choice, weights and the experts' rows against the plain functions; rows of a token do not depend on the
    tokens beside it."""
    from cie_amd.kernels import ops

    T, E, top, width, ff = sizes
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, width, generator=g).to(dtype)
    logits = torch.randn(T, E, generator=g) * 2
    w = {f"e{e}.{n}": (torch.randn(*s, generator=g) * 1.5 / s[1] ** 0.5).to(dtype).float()
         for e in range(E) for n, s in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff)))}
    gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(dtype).cuda()
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(dtype).cuda()
    mfma = dtype == torch.bfloat16 and width % 8 == 0 and ff % 8 == 0
    for tile_rows in ((16, 32, 64, 128) if mfma else (16, 5)):
        route = ops.experts_route(logits.cuda(), top, tile_rows)
        scores = torch.sigmoid(logits)
        want_w, want_e = torch.topk(scores, top, dim=1)
        assert torch.equal(route.pair_expert.cpu().reshape(T, top).long(), want_e)
        assert torch.allclose(route.pair_weight.cpu().reshape(T, top), want_w, atol=1e-6)
        order = route.sorted.cpu().long()
        assert sorted(order.tolist()) == list(range(T * top))
        assert bool((route.pair_expert.cpu().long()[order].diff() >= 0).all())        # sorted by expert
        n = int(route.n_tiles.cpu())
        assert n <= route.max_tiles and int(route.tile_count.cpu()[:n].sum()) == T * top
        parts = ops.experts_forward(x.cuda(), route, gate_up, down, 1.25, 1.702, 1.0, mfma=mfma).cpu().double()
        tol = 2e-5 if dtype == torch.float32 else 3e-2
        for t in range(0, T, max(1, T // 25)):
            for j in range(top):
                scaled = (want_w[t, j] * x[t].float()).to(dtype).double()
                want = pg.expert(pg.cast(w, torch.float64), f"e{int(want_e[t, j])}.", scaled[None], 1.25)[0]
                assert torch.allclose(parts[t, j], want, atol=tol, rtol=tol), (t, j, tile_rows)
    alone = ops.experts_forward(x[:1].cuda().contiguous(), ops.experts_route(logits[:1].cuda().contiguous(), top, 16),
                                gate_up, down, 1.25, 1.702, 1.0, mfma=mfma).cpu().double()
    if dtype == torch.float32:
        assert torch.equal(alone[0], parts[0])
    else:  # (few tiles split K over the waves: the same sums in another order, and a bfloat16 rounding may turn)
        assert torch.allclose(alone[0], parts[0], atol=1e-2, rtol=1e-2)


def test_routing_of_large_and_of_equal_logits():
    """Logits so large that their scores round to 1 are still ranked; equal logits go to the lower index; logits of
    minus infinity are chosen last, and with a score of zero."""
    from cie_amd.kernels import ops

    logits = torch.tensor([[20.0, 45.0, 30.0, 25.0, 45.5, -3.0],
                           [1.0, 2.0, 2.0, 0.5, 2.0, 1.5],
                           [float("-inf"), -100.0, float("-inf"), -95.0, float("-inf"), float("-inf")]])
    route = ops.experts_route(logits.cuda(), 4, 16)
    assert route.pair_expert.cpu().reshape(3, 4).tolist() == [[4, 1, 2, 3], [1, 2, 4, 5], [3, 1, 0, 2]]
    weights = route.pair_weight.cpu().reshape(3, 4)
    assert torch.equal(weights[0], torch.ones(4)) and torch.allclose(weights[1], torch.sigmoid(torch.tensor([2.0, 2.0, 2.0, 1.5])))
    assert bool((weights[2] == 0).all())
    wide = torch.zeros(2, 200)
    wide[0, 131], wide[0, 64], wide[1, 199] = 3.0, 3.0, -1.0
    assert ops.experts_route(wide.cuda(), 3, 16).pair_expert.cpu().reshape(2, 3).tolist() == [[64, 131, 0], [0, 1, 2]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(dtype):
    """The branch's norm and add (with the rows of a sum), the bounded unit, the smooth bound, the scaled embedding."""
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(2)
    for rows, hidden, n_parts in ((3, 40, 0), (70, 192, 2), (9, 2048, 4)):
        residual = torch.randn(rows, hidden, generator=g)
        branch = torch.randn(rows, hidden, generator=g).to(dtype)
        parts = torch.randn(rows, max(n_parts, 1), hidden, generator=g)
        weight = 1.0 + 0.3 * torch.randn(hidden, generator=g)
        stream = residual.clone().cuda()
        out = ops.branch_norm_add(stream, branch.cuda(), weight.cuda(), 1e-5, dtype, parts=parts.cuda() if n_parts else None)
        y = branch.double() + (parts.double().sum(1) if n_parts else 0)
        want = residual.double() + y / pg.rms(y, 1e-5) * weight.double()
        assert torch.allclose(stream.double().cpu(), want, atol=2e-5)
        assert torch.allclose(out.double().cpu(), want, atol=1e-5 if dtype == torch.float32 else 0, rtol=0 if dtype == torch.float32 else 1e-2)
        only_parts = residual.clone().cuda()
        ops.branch_norm_add(only_parts, None, weight.cuda(), 1e-5, dtype, parts=parts.cuda(), want_rows=False)
        y = parts.double().sum(1)
        assert torch.allclose(only_parts.double().cpu(), residual.double() + y / pg.rms(y, 1e-5) * weight.double(), atol=2e-5)
    gate_up = (torch.randn(11, 2 * 37, generator=g) * 3).to(dtype)
    got = ops.clamped_glu(gate_up.cuda(), 1.5, 1.702, 1.0).double().cpu()
    gate, up = gate_up[:, :37].double().clamp(max=1.5), gate_up[:, 37:].double().clamp(-1.5, 1.5)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got, gate * torch.sigmoid(1.702 * gate) * (up + 1), atol=tol, rtol=tol)
    if dtype == torch.float32:
        x = torch.randn(5, 33, generator=g) * 40
        assert torch.allclose(ops.soft_cap_(x.clone().cuda(), 15.0).cpu(), 15.0 * torch.tanh(x / 15.0), atol=1e-5)
    table = torch.randn(20, 24, generator=g).to(dtype).cuda()
    ids = torch.tensor([3, 19, 0], dtype=torch.int32).cuda()
    rows = torch.empty(3, 24, dtype=dtype).cuda()
    out = ops.embed(table, ids, scale=0.5, rows=rows)
    assert torch.equal(out, table[ids.long()].float() * 0.5) and torch.equal(rows, (table[ids.long()].float() * 0.5).to(dtype))
