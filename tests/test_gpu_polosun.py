"""GPU: the Polosun decoder in the engine against the plain implementation (tests/plain_polosun.py): every
mechanism alone, every way of cutting and batching the same requests, reused pages and slots, long prompts and long
decoding, other sizes, and greedy generation through the engine's own entry point."""

from __future__ import annotations

import random

import numpy as np
import pytest
import torch

import plain_polosun
import polosun_util as pu
import replay_util
from conftest import random_tokens

pytestmark = pytest.mark.gpu

# a row's error is the root mean square of the difference of its logits, mean taken off, as a share of the
# logits' own spread.  float32: sums in another order; this is the sharp test of cache, state and batching.
# bfloat16: activations rounded to 8 bits between kernels, with these bold weights (peaked softmax, branches
# weighed up to 1.25) a few per cent at the worst row and under two on average (RMS_LIMIT).
LIMIT = {"float32": 2e-5, "bfloat16": 8e-2}
RMS_LIMIT = {"float32": 1e-5, "bfloat16": 3e-2}


def plain_all(raw, weights, requests):
    return {rid: plain_polosun.forward(raw, weights, tokens).float() for rid, tokens in requests.items()}


def run_and_compare(raw, weights, requests, steps, dtype, plain, page_size=16, max_running=4, limit=None):
    pool = max(replay_util.max_live_tokens(steps, page=page_size), page_size)
    runner = pu.make_runner(raw, weights, dtype, pool, page_size, max_running)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    for rid in requests:
        assert rid in rows, f"{rid}: no logits"
    worst, rms = pu.spread(rows, plain)
    assert worst <= (limit or LIMIT[dtype]) and rms <= RMS_LIMIT[dtype], (dtype, worst, rms)
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0
    return rows


MECHANISMS = {
    "latent_attention": {"type": "latent_attention", "mlp": None,
                         "mixer": {"heads": 2, "dim": 8, "rot_dim": 8, "vdim": 12, "kv_rank": 20, "scale": 0.7,
                                   "rot": {"base": 200.0, "dims": 8}}},
    "latent_attention_stretched": {"type": "latent_attention", "mlp": None,
                                   "mixer": {"heads": 4, "dim": 12, "rot_dim": 16, "vdim": 4, "kv_rank": 8, "scale": 0.5,
                                             "rot": {"base": 1000.0, "dims": 16, "scaling":
                                                     {"factor": 8.0, "fast": 8.0, "original": 32, "slow": 0.5}}}},
    "latent_attention_unturned": {"type": "latent_attention", "mlp": None,
                                  "mixer": {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 8, "kv_rank": 12, "scale": 0.9}},
    "retention": {"type": "retention", "mlp": None,
                  "mixer": {"heads": 2, "dim": 12, "vdim": 20, "decay": [0.875, 0.99609375], "rot": {"base": 300.0, "dims": 12}}},
    "retention_part_turned": {"type": "retention", "mlp": None,
                              "mixer": {"heads": 3, "dim": 40, "vdim": 8, "decay": [0.5, 0.9, 0.999], "rot": {"base": 20.0, "dims": 6}}},
    "retention_unturned": {"type": "retention", "mlp": None, "mixer": {"heads": 1, "dim": 4, "vdim": 72, "decay": [0.96875]}},
    "rglru": {"type": "rglru", "mlp": None, "mixer": {"width": 40, "blocks": 5, "conv": 3}},
    "rglru_one_tap": {"type": "rglru", "mlp": None, "mixer": {"width": 16, "blocks": 1, "conv": 1}},
    "rglru_long_taps": {"type": "rglru", "mlp": None, "mixer": {"width": 24, "blocks": 2, "conv": 7}},
    "feed_forward": {"type": "rglru", "mlp": {"kind": "dense", "ff": 44}, "mixer": {"width": 8, "blocks": 1, "conv": 2}},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_a_mechanism_alone(name, dtype):
    """One layer of one kind: whole prompts, then the same tokens in portions down to two tokens and one by one
    (shorter than the convolution's reach, across pages), two requests side by side."""
    raw = pu.single(MECHANISMS[name])
    weights = pu.make_weights(raw, seed=3)
    requests = {"a": random_tokens(45, raw["vocab"], 1), "b": random_tokens(21, raw["vocab"], 2), "c": [7]}
    plain = plain_all(raw, weights, requests)
    run_and_compare(raw, weights, requests, replay_util.whole(requests), dtype, plain)
    run_and_compare(raw, weights, requests, replay_util.portions(requests, sizes=(2, 3, 2, 17, 2, 5)), dtype, plain)
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, chunk_sizes=(2, 7, 3), decode_tail=9),
                    dtype, plain, max_running=3)


SCHEDULES = {
    "whole": replay_util.whole,
    "tail": lambda requests: replay_util.tail_one_by_one(requests, tail=20),
    "portions": replay_util.portions,
    "mixed": lambda requests: replay_util.mixed(requests, live=4),
}
LENGTHS = {"A": [5, 17, 33, 70, 100, 1], "B": [2, 9, 40, 64, 131]}


@pytest.fixture(scope="module")
def models():
    out = {}
    for index, (name, raw) in enumerate(pu.SMALL.items()):
        weights = pu.make_weights(raw, seed=20 + index)
        requests = {f"{name}{i}": random_tokens(n, raw["vocab"], seed=50 + i) for i, n in enumerate(LENGTHS[name])}
        out[name] = (raw, weights, requests, plain_all(raw, weights, requests))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("name", sorted(pu.SMALL))
def test_logits_do_not_depend_on_cutting_or_batching(models, name, schedule, dtype):
    """Prefill against token-by-token decoding, portions of several sizes, unequal requests in one batch against
    each alone; six requests take turns on four slots, and the pool is no larger than the schedule's peak."""
    raw, weights, requests, plain = models[name]
    run_and_compare(raw, weights, requests, SCHEDULES[schedule](requests), dtype, plain)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(pu.SMALL))
def test_captured_steps_give_the_same_logits(models, name, dtype):
    """Steps of single tokens replay captured graphs (and short mixed steps theirs, from the second time a shape
    comes), with uncaptured steps between the replays: every replay is checked against the plain logits, and states
    move on once per token although a capture runs the kernels on rows of padding."""
    raw, weights, requests, plain = models[name]
    steps = replay_util.fixed_portions(requests, portion=8, live=3, decode_tail=14)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = pu.make_runner(raw, weights, dtype, pool, 16, 4, graph_decode=True)
    assert runner.graphs is not None, "the model's parts all say that they may be captured"
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    worst, rms = pu.spread(rows, plain)
    assert runner.graph_replays >= 10 and runner.mixed_graph_replays > 0, (runner.graph_replays, runner.mixed_graph_replays)
    assert worst <= LIMIT[dtype] and rms <= RMS_LIMIT[dtype], (worst, rms)


@pytest.mark.parametrize("page_size", [4, 64])
def test_other_page_sizes(models, page_size):
    raw, weights, requests, plain = models["A"]
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=5), "float32", plain,
                    page_size=page_size, max_running=3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_traces_reuse_pages_and_slots(models, dtype):
    """Random cuts (one token, two, up to a page's edge, one past it) of ten requests on three slots: every slot
    and page is handed out again, and a state that a new request found uncleared would show at its first token."""
    raw, weights, _, _ = models["B"]
    rng = random.Random(4)
    requests, steps = replay_util.random_trace(rng, [3, 40, 17, 1, 33, 64, 2, 18, 49, 31], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    wanted = {rid: {pos: None for pos in range(len(tokens))} for rid, tokens in requests.items()}
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = pu.make_runner(raw, weights, dtype, pool, 16, 3)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert set(rows) <= set(wanted) and rows
    worst, _ = pu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


NEEDLE, ASK, FILLERS = 1, 2, 40  # token ids: the one to be found, the one that looks for it, the first of the rest


def planted(kind: str):
    """A single layer whose weights are changed by hand so that one score stands out: the token ASK looks, through a
    query dimension that only it has, for a key dimension that only the token NEEDLE has, wherever that lies."""
    if kind == "latent_attention":
        layer = {"type": "latent_attention", "mlp": None,
                 "mixer": {"heads": 2, "dim": 16, "rot_dim": 8, "vdim": 16, "kv_rank": 24, "scale": 0.25,
                           "rot": {"base": 10000.0, "dims": 8}}}
    else:
        layer = {"type": "retention", "mlp": None,
                 "mixer": {"heads": 2, "dim": 16, "vdim": 16, "decay": [0.998046875, 0.9990234375],
                           "rot": {"base": 10000.0, "dims": 8}}}
    raw = pu.single(layer, width=32, vocab=64)
    w = pu.make_weights(raw, seed=9)
    w["embed"][:, 0:2] = 0.0
    w["embed"][NEEDLE, 0] = 8.0
    w["embed"][ASK, 1] = 8.0
    heads, dim = layer["mixer"]["heads"], layer["mixer"]["dim"]
    if kind == "latent_attention":
        per = dim + layer["mixer"]["rot_dim"]
        w["l0.mix.dkv"][:, 0:2] = 0.0
        w["l0.mix.dkv"][0, :] = 0.0
        w["l0.mix.dkv"][0, 0] = 4.0            # latent 0 is the needle's mark
        w["l0.mix.uk"][:, 0] = 0.0
        w["l0.mix.q"][:, 0:2] = 0.0
        for h in range(heads):
            w["l0.mix.uk"][h * dim, :] = 0.0
            w["l0.mix.uk"][h * dim, 0] = 4.0    # plain key dimension 0 of every head reads it
            w["l0.mix.q"][h * per, :] = 0.0
            w["l0.mix.q"][h * per, 1] = 4.0     # plain query dimension 0 of every head reads the asker's mark
    else:
        at = 12                                 # a dimension that does not turn
        for name, column in (("k", 0), ("q", 1)):
            w["l0.mix." + name][:, 0:2] = 0.0
            for h in range(heads):
                w["l0.mix." + name][h * dim + at, :] = 0.0
                w["l0.mix." + name][h * dim + at, column] = 16.0
    w["l0.mix.o"] *= 4.0                        # the layer's branch outweighs the embedding's own share of the logits
    return raw, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["latent_attention", "retention"])
def test_one_key_among_hundreds_is_found_wherever_it_lies(kind, dtype):
    """The needle at the first positions, at page borders, far back; asked for inside a prompt's portion and by a
    token decoded alone, across several requests that share a pool and reuse slots.  A lost key, a key of a wrong
    page or slot, or a state that is not carried moves these logits by far more than the tolerance (checked below
    on the plain implementation itself)."""
    raw, weights = planted(kind)
    length = 600
    places = [0, 1, 15, 16, 17, 63, 64, 300, 511, 512, 590]
    requests = {}
    for place in places:
        tokens = [FILLERS + t % (raw["vocab"] - FILLERS) for t in random_tokens(length, 1000, 30 + place)]
        tokens[place] = NEEDLE
        requests[f"n{place}"] = tokens + [ASK, FILLERS, ASK]
    plain = plain_all(raw, weights, requests)
    # the test of the test: without the needle the asked rows are far off
    for rid in ("n0", "n300"):
        blind = list(requests[rid])
        blind[blind.index(NEEDLE)] = FILLERS + 3
        other = plain_polosun.forward(raw, weights, blind).float()
        for row in (length, length + 2):
            diff = other[row] - plain[rid][row]
            assert float((diff - diff.mean()).pow(2).mean().sqrt() / plain[rid][row].std()) > 0.5
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
    runner = pu.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == [length, length + 1, length + 2] for rid in requests)
    worst, _ = pu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A prompt of 300 tokens, then 250 tokens decoded one by one across page borders, every layer kind in the model."""
    raw = pu.SMALL_A
    weights = pu.make_weights(raw, seed=31)
    requests = {"long": random_tokens(550, raw["vocab"], 7)}
    stepper = plain_polosun.Stepper(raw, weights)
    plain = {"long": torch.stack([stepper.token(t) for t in requests["long"]]).float()}
    steps = replay_util.tail_one_by_one(requests, tail=250)
    run_and_compare(raw, weights, requests, steps, dtype, plain, max_running=1)


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
        engine.model.load(pu.Fixed(weights), dtype, "cuda:0")
        results = engine.generate(prompts, GenerationConfig(max_output_tokens=12))
        for prompt, result in zip(prompts, results):
            assert len(result.token_ids) == 12
            turned = replay_util.greedy_tokens_follow_plain(
                lambda tokens: plain_polosun.forward(raw, weights, tokens), prompt, result.token_ids,
                (lambda tokens: plain_polosun.forward(raw, weights, tokens, dtype=torch.bfloat16)) if dtype == "bfloat16" else None)
            assert turned <= (0 if dtype == "float32" else 3)


def test_the_trace_runner_replays_a_model_folder(tmp_path, models):
    """bin/trace_run on a folder written for it: same logits as the plain implementation, four slots by default."""
    import json
    import subprocess
    import sys

    from cie_amd.weights import write_tensors
    from conftest import ROOT

    raw, weights, requests, plain = models["B"]
    folder = write_tensors(tmp_path / "model", raw, {k: v.to(torch.bfloat16) for k, v in weights.items()})
    steps = replay_util.mixed(requests, live=4)
    out = tmp_path / "out"
    pool = replay_util.max_live_tokens(steps, page=64)
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", str(pool)],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.split("\n") if line.startswith("done")] == [f"done {s['step']}" for s in steps]
    outputs = {s["step"]: np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, raw["vocab"])
               for s in steps if any(e["want"] for e in s["entries"])}
    worst, _ = pu.spread(replay_util.by_position(steps, outputs), plain)
    assert worst <= LIMIT["float32"], worst


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 7, 16, 17, 64, 150])
def test_block_diagonal_product_in_all_its_forms(rows, dtype):
    """Few rows, tiles, and (bfloat16) the matrix cores; blocks read from and written to columns of wider rows, with
    bias, with a sigmoid gate, float32 results from bfloat16 operands; a K that is no multiple of 32, and one that is
    no multiple of 8 (which keeps off the matrix cores)."""
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(rows)
    for blocks, n, k, a_block, extra in ((3, 24, 40, 56, 8), (2, 80, 96, 96, 0), (5, 17, 12, 20, 4)):
        a = torch.randn(rows, extra + (blocks - 1) * a_block + k + 3, generator=g).to(dtype).cuda()
        w = (torch.randn(blocks, n, k, generator=g) / k ** 0.5).to(dtype).cuda()
        bias = torch.randn(blocks, n, generator=g).to(dtype).cuda()
        gate = torch.randn(rows, 5 + blocks * n, generator=g).to(dtype).cuda()
        picked = torch.stack([a[:, extra + b * a_block: extra + b * a_block + k] for b in range(blocks)], 1).double()
        plain = torch.einsum("mbk,bnk->mbn", picked, w.double())
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        out = ops.block_linear(a, w, a_block=a_block, a_offset=extra, out_dtype=torch.float32)
        assert torch.allclose(out.double().reshape(rows, blocks, n), plain, atol=2e-5 if dtype == torch.float32 else 1e-4)
        with_bias = ops.block_linear(a, w, bias, a_block=a_block, a_offset=extra)
        assert with_bias.dtype == dtype
        assert torch.allclose(with_bias.double().reshape(rows, blocks, n), plain + bias.double(), atol=tol, rtol=tol)
        wide = torch.full((rows, 6 + blocks * (n + 2)), 7.0, dtype=dtype, device="cuda")
        ops.block_linear(a, w, a_block=a_block, a_offset=extra, out=wide, out_offset=6, c_block=n + 2, gate=gate, gate_offset=5)
        gated = plain * torch.sigmoid(gate[:, 5:].double().reshape(rows, blocks, n))
        got = wide[:, 6:].reshape(rows, blocks, n + 2)
        assert torch.allclose(got[:, :, :n].double(), gated, atol=tol, rtol=tol)
        assert bool((wide[:, :6] == 7).all()) and bool((got[:, :-1, n:] == 7).all())  # nothing beside the blocks is touched
    # a row's result does not depend on the rows beside it
    if 1 < rows <= 4 or (dtype == torch.float32 and rows <= 16):  # (within one form of the kernel, bit for bit)
        alone = ops.block_linear(a[:1].contiguous(), w, a_block=a_block, a_offset=extra, out_dtype=torch.float32)
        assert torch.equal(alone, out[:1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_boundary_kernel(dtype):
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(1)
    for rows, hidden in ((3, 40), (130, 1024), (9, 2048)):
        history = torch.randn(5, rows, hidden, generator=g).cuda()
        x = torch.randn(rows, hidden, generator=g).cuda()
        a = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
        b = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
        weights = torch.randn(4, generator=g).cuda()
        kept = history.clone()
        stream, normed = ops.depth_stream(x, a, b, mult=0.7, history=history, newest=3, weights=weights, gains=(1.5, 0.25),
                                          out_dtype=dtype, eps=1e-5)
        new = x.double() + 0.7 * (a.double() + b.double())
        assert torch.allclose(history[3].double(), new, atol=1e-5) and torch.equal(history[[0, 1, 2, 4]], kept[[0, 1, 2, 4]])
        want = sum(weights[j].double() * (new if j == 3 else kept[j].double()) for j in range(4))
        assert torch.allclose(stream.double(), want, atol=2e-5)
        unit = want / torch.sqrt((want * want).mean(-1, keepdim=True) + 1e-5)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(normed[0].double(), unit * 1.5, atol=tol, rtol=tol)
        assert torch.allclose(normed[1].double(), unit * 0.25, atol=tol, rtol=tol)
        # one branch, no average, one norm; and norms alone
        stream, normed = ops.depth_stream(x, a, mult=2.0, gains=(1.0,), out_dtype=dtype, eps=1e-5)
        assert torch.allclose(stream.double(), x.double() + 2.0 * a.double(), atol=1e-5) and len(normed) == 1
        nothing, normed = ops.depth_stream(x, gains=(3.0, 1.0), out_dtype=dtype, eps=1e-5, want_stream=False)
        unit = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5)
        assert nothing is None and torch.allclose(normed[0].double(), 3.0 * unit, atol=tol, rtol=tol)
