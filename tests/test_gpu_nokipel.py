"""GPU: the Nokipel decoder in the engine against the plain implementation (tests/plain_nokipel.py): every
mechanism alone, every way of cutting and batching the same requests, reused pages and slots, keys at the edges of
chunks and far back, long decoding, other sizes, and greedy generation through the engine's own entry point."""

from __future__ import annotations

import copy
import functools
import random

import numpy as np
import pytest
import torch

import nokipel_util as nu
import plain_nokipel as pn
import replay_util
from conftest import random_tokens

pytestmark = pytest.mark.gpu

# a row's error is the root mean square of the difference of its logits, mean taken off, as a share of the
# logits' own spread.  float32: sums in another order; this is the sharp test of cache, state and batching.
# bfloat16: activations rounded to 8 bits between kernels, with these bold weights a few per cent at the worst row.
LIMIT = {"float32": 2e-5, "bfloat16": 8e-2}
RMS_LIMIT = {"float32": 1e-5, "bfloat16": 3e-2}


def plain_all(raw, weights, requests):
    return {rid: pn.forward(raw, weights, tokens).float() for rid, tokens in requests.items()}


def run_and_compare(raw, weights, requests, steps, dtype, plain, page_size=16, max_running=4, limit=None, graph_decode=False):
    pool = max(replay_util.max_live_tokens(steps, page=page_size), page_size)
    runner = nu.make_runner(raw, weights, dtype, pool, page_size, max_running, graph_decode=graph_decode)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    for rid in requests:
        assert rid in rows, f"{rid}: no logits"
    worst, rms = nu.spread(rows, plain)
    assert worst <= (limit or LIMIT[dtype]) and rms <= RMS_LIMIT[dtype], (dtype, worst, rms)
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0
    return rows


TINY_MIXER = {"heads": 1, "dim": 4, "vdim": 4, "decay": [0.5]}
MOE_FULL = {"kind": "moe", "router": {"experts": 6, "identity": 2, "top": 3, "scale": 2.5, "groups": {"count": 4, "keep": 2}},
            "expert": {"ff": 24}, "shared": {"ff": 16}}

MECHANISMS = {
    # a rotation over half of the head, chunks that end inside pages, two query heads a key head
    "attention": {"type": "attention", "mlp": None,
                  "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.4, "mask": {"size": 7},
                            "rot": {"base": 200.0, "dims": 8}}},
    # every number turns; one key head for all; chunks as long as a page
    "attention_all_turned": {"type": "attention", "mlp": None,
                             "mixer": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 24, "scale": 0.6, "mask": {"size": 16},
                                       "rot": {"base": 1000.0, "dims": 8}}},
    # chunks of two tokens: every other token sees itself alone; every query head its own key head
    "attention_pairs_of_tokens": {"type": "attention", "mlp": None,
                                  "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 24, "scale": 0.3, "mask": {"size": 2},
                                            "rot": {"base": 30.0, "dims": 6}}},
    "attention_alone_in_its_chunk": {"type": "attention", "mlp": None,
                                     "mixer": {"heads": 2, "dim": 8, "vdim": 8, "scale": 0.3, "mask": {"size": 1},
                                               "rot": {"base": 30.0, "dims": 2}}},
    # no chunks, no rotation, no kv_heads in the file
    "attention_plain": {"type": "attention", "mlp": None, "mixer": {"heads": 2, "dim": 12, "vdim": 20, "scale": 0.5}},
    # head sizes of the matrix-core kernels
    "attention_heads_of_64": {"type": "attention", "mlp": None,
                              "mixer": {"heads": 6, "kv_heads": 3, "dim": 64, "vdim": 64, "scale": 0.15, "mask": {"size": 33},
                                        "rot": {"base": 300000.0, "dims": 32}}},
    "attention_heads_of_128_and_64": {"type": "attention", "mlp": None,
                                      "mixer": {"heads": 2, "kv_heads": 1, "dim": 128, "vdim": 64, "scale": 0.1,
                                                "mask": {"size": 40}, "rot": {"base": 10000.0, "dims": 128}}},
    "lightning": {"type": "lightning", "mlp": None,
                  "mixer": {"heads": 2, "dim": 12, "vdim": 20, "decay": [0.875, 0.99609375]}},
    "lightning_one_head": {"type": "lightning", "mlp": None, "mixer": {"heads": 1, "dim": 4, "vdim": 72, "decay": [0.96875]}},
    "lightning_wide_keys": {"type": "lightning", "mlp": None,
                            "mixer": {"heads": 3, "dim": 40, "vdim": 8, "decay": [0.5, 0.9, 0.999]}},
    "lightning_heads_of_64": {"type": "lightning", "mlp": None,
                              "mixer": {"heads": 2, "dim": 64, "vdim": 64, "decay": [0.75, 0.998046875]}},
    # keys of more than 64 and of more than 128 numbers: more tiles of the memory's rows a wave in the walk by blocks
    "lightning_heads_of_128": {"type": "lightning", "mlp": None,
                               "mixer": {"heads": 2, "dim": 128, "vdim": 128, "decay": [0.9375, 0.99951171875]}},
    "lightning_long_keys": {"type": "lightning", "mlp": None,
                            "mixer": {"heads": 1, "dim": 160, "vdim": 24, "decay": [0.984375]}},
    # keys too long for the walk by blocks: prompts walk token by token
    "lightning_keys_beyond_the_blocks": {"type": "lightning", "mlp": None,
                                         "mixer": {"heads": 2, "dim": 168, "vdim": 16, "decay": [0.9375, 0.9990234375]}},
    # rows of all heads' read-outs wider than one wave norms: 1,080 and 2,176 numbers
    "lightning_wide_rows": {"type": "lightning", "mlp": None,
                            "mixer": {"heads": 9, "dim": 4, "vdim": 120, "decay": [0.5 + 0.055 * h for h in range(9)]}},
    "lightning_many_heads": {"type": "lightning", "mlp": None,
                             "mixer": {"heads": 17, "dim": 8, "vdim": 128, "decay": [1.0 - 2.0 ** -(1 + h % 9) for h in range(17)]}},
    "dense": {"type": "lightning", "mixer": TINY_MIXER, "mlp": {"kind": "dense", "ff": 44, "limit": 0.5}},
    "dense_wide_limit": {"type": "lightning", "mixer": TINY_MIXER, "mlp": {"kind": "dense", "ff": 20, "limit": 30.0}},
    "experts": {"type": "lightning", "mixer": TINY_MIXER, "mlp": MOE_FULL},
    # no groups, no identity experts, no shared expert, no scale in the file
    "experts_plain": {"type": "lightning", "mixer": TINY_MIXER,
                      "mlp": {"kind": "moe", "router": {"experts": 5, "top": 2}, "expert": {"ff": 40}}},
    "experts_mostly_identity": {"type": "lightning", "mixer": TINY_MIXER,
                                "mlp": {"kind": "moe", "router": {"experts": 1, "identity": 3, "top": 2, "scale": 0.75,
                                                                  "groups": {"count": 2, "keep": 1}},
                                        "expert": {"ff": 8}, "shared": {"ff": 8}}},
    "experts_all_chosen": {"type": "lightning", "mixer": TINY_MIXER,
                           "mlp": {"kind": "moe", "router": {"experts": 3, "identity": 1, "top": 4, "scale": 1.0,
                                                             "groups": {"count": 2, "keep": 2}},
                                   "expert": {"ff": 16}}},
    "experts_one_chosen": {"type": "lightning", "mixer": TINY_MIXER,
                           "mlp": {"kind": "moe", "router": {"experts": 9, "top": 1, "scale": 3.0, "groups": {"count": 3, "keep": 1}},
                                   "expert": {"ff": 16}, "shared": {"ff": 40}}},
}
LOOPS = {
    "loop_of_one_layer": ({"type": "lightning", "mlp": {"kind": "dense", "ff": 24, "limit": 1.0},
                           "mixer": {"heads": 2, "dim": 8, "vdim": 8, "decay": [0.75, 0.96875]}}, {"start": 0, "stop": 1, "times": 3}),
    "loop_of_attention": ({"type": "attention", "mlp": MOE_FULL,
                           "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.4, "mask": {"size": 9},
                                     "rot": {"base": 50.0, "dims": 4}}}, {"start": 0, "stop": 1, "times": 2}),
}


def mechanism(name: str) -> dict:
    if name in LOOPS:
        layer, loop = LOOPS[name]
        return nu.single(copy.deepcopy(layer), loop=loop)
    return nu.single(copy.deepcopy(MECHANISMS[name]))


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS) + sorted(LOOPS))
def test_a_mechanism_alone(name, dtype):
    """One layer of one kind: whole prompts, then the same tokens in portions down to two tokens and one by one
    (across pages and chunks), requests side by side.  Routers read the whole stream in float32 and markers in
    bfloat16, where a near-tie could turn."""
    raw = mechanism(name)
    weights = nu.make_weights(raw, seed=3, exact_router=dtype == "bfloat16")
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
    for index, (name, raw) in enumerate(nu.SMALL.items()):
        weights = nu.make_weights(raw, seed=20 + index, exact_router=True)
        requests = {f"{name}{i}": random_tokens(n, raw["vocab"], seed=50 + i) for i, n in enumerate(LENGTHS[name])}
        out[name] = (raw, weights, requests, plain_all(raw, weights, requests))
    return out


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("name", sorted(nu.SMALL))
def test_logits_do_not_depend_on_cutting_or_batching(models, name, schedule, dtype):
    """Prefill against token-by-token decoding, portions of several sizes, unequal requests in one batch against
    each alone; more requests than slots take turns, and the pool is no larger than the schedule's peak."""
    raw, weights, requests, plain = models[name]
    run_and_compare(raw, weights, requests, SCHEDULES[schedule](requests), dtype, plain)


def test_routers_that_read_the_whole_stream(models):
    """Float32, weights without markers: routers, corrections and groups on ordinary rows."""
    for name, (raw, _, requests, _) in models.items():
        weights = nu.make_weights(raw, seed=40)
        plain = plain_all(raw, weights, requests)
        run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=2), "float32", plain, max_running=3)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(nu.SMALL))
def test_captured_steps_give_the_same_logits(models, name, dtype):
    """Steps of single tokens replay captured graphs (and short mixed steps theirs, from the second time a shape
    comes), with uncaptured steps between the replays: every replay is checked against the plain logits, and
    memories move on once per token although a capture runs the kernels on rows of padding."""
    raw, weights, requests, plain = models[name]
    steps = replay_util.fixed_portions(requests, portion=8, live=3, decode_tail=14)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = nu.make_runner(raw, weights, dtype, pool, 16, 4, graph_decode=True)
    assert runner.graphs is not None, "the model's parts all say that they may be captured"
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    worst, rms = nu.spread(rows, plain)
    assert runner.graph_replays >= 10 and runner.mixed_graph_replays > 0, (runner.graph_replays, runner.mixed_graph_replays)
    assert worst <= LIMIT[dtype] and rms <= RMS_LIMIT[dtype], (worst, rms)


@pytest.mark.parametrize("page_size", [4, 64])
def test_other_page_sizes(models, page_size):
    raw, weights, requests, plain = models["A"]
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=5), "float32", plain,
                    page_size=page_size, max_running=3)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(nu.SMALL))
def test_random_traces_reuse_pages_and_slots(models, name, dtype):
    """Random cuts (one token, two, up to a page's edge, one past it) of ten requests on three slots: every slot
    and page is handed out again, and a memory that a new request found uncleared would show at its first token."""
    raw, weights, _, _ = models[name]
    rng = random.Random(4)
    requests, steps = replay_util.random_trace(rng, [3, 40, 17, 1, 33, 64, 2, 18, 49, 31], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = nu.make_runner(raw, weights, dtype, pool, 16, 3)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert set(rows) <= set(requests) and rows
    worst, _ = nu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


def random_configuration(rng: random.Random) -> dict:
    """A model whose every size, count, constant and layer order is drawn: widths and heads that are and are not
    multiples of 8 or 64, chunks shorter than a page and longer than any request, loops anywhere."""
    groups = rng.choice([2, 3, 4, 6])
    width = groups * rng.choice([8, 12, 16, 20, 32])
    layers = []
    for _ in range(rng.randint(2, 6)):
        if rng.random() < 0.5:
            heads = rng.choice([1, 2, 3, 5])
            mixer = {"heads": heads, "dim": rng.choice([4, 8, 24, 64, 72, 136]), "vdim": rng.choice([8, 16, 40, 64, 128]),
                     "decay": [rng.choice([0.25, 0.75, 0.9375, 0.99609375, 0.9990234375]) for _ in range(heads)]}
            kind = "lightning"
        else:
            kv_heads = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 24, 64, 128])
            mixer = {"heads": kv_heads * rng.choice([1, 2, 4]), "kv_heads": kv_heads, "dim": dim,
                     "vdim": rng.choice([8, 24, 64, 128]), "scale": rng.choice([0.5, 1.0, 2.0]) * dim ** -0.5,
                     "mask": {"size": rng.choice([1, 3, 16, 17, 31, 64, 500])},
                     "rot": {"base": rng.choice([10.0, 1000.0, 2.0e5]), "dims": rng.choice([d for d in (2, 4, 8, 16, 64, 128) if d <= dim])}}
            kind = "attention"
        draw = rng.random()
        if draw < 0.15:
            mlp = None
        elif draw < 0.5:
            mlp = {"kind": "dense", "ff": rng.choice([24, 52, 100]), "limit": rng.choice([0.5, 1.0, 4.0])}
        else:
            count, per = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 5])
            outputs = count * per
            identity = rng.randint(0, min(outputs - 1, 3))
            keep = rng.randint(1, count)
            mlp = {"kind": "moe", "expert": {"ff": rng.choice([8, 20, 48])}, "shared": {"ff": rng.choice([8, 28])},
                   "router": {"experts": outputs - identity, "identity": identity, "top": rng.randint(1, min(keep * per, 6)),
                              "scale": rng.choice([0.5, 1.0, 2.5]), "groups": {"count": count, "keep": keep}}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    start = rng.randint(0, len(layers) - 1)
    return {"architecture": "Nokipel", "vocab": rng.choice([70, 130, 300]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3]), "groups": groups}, "embedding": {"scale": rng.choice([0.5, 2.0, 8.0])},
            "loop": {"start": start, "stop": rng.randint(start, len(layers)), "times": rng.randint(1, 3)}, "layers": layers}


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations_and_traces(seed):
    """Ten models that nobody chose, each under a random trace of six requests on three slots, in both precisions."""
    rng = random.Random(1000 + seed)
    raw = random_configuration(rng)
    weights = nu.make_weights(raw, seed=seed, exact_router=True)
    requests, steps = replay_util.random_trace(rng, [rng.choice([1, 2, 9, 33, 48, 70]) for _ in range(6)], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    for dtype in ("float32", "bfloat16"):
        runner = nu.make_runner(raw, weights, dtype, max(replay_util.max_live_tokens(steps, page=16), 16), 16, 3)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        assert rows
        worst, _ = nu.spread(rows, plain)
        assert worst <= LIMIT[dtype], (dtype, worst, raw)
        assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0


NEEDLE, ASK, FILLERS = 1, 2, 40  # token ids: the one to be found, the one that looks for it, the first of the rest
CHUNK = 200
AT = 12                          # the head's number that carries the mark: one that does not turn


def planted(kind: str):
    """A single layer whose weights are changed by hand so that one score stands out: the token ASK looks, through a
    query number that only it has, for a key number that only the token NEEDLE has, wherever that lies."""
    if kind == "lightning":
        layer = {"type": "lightning", "mlp": None,
                 "mixer": {"heads": 2, "dim": 16, "vdim": 16, "decay": [0.998046875, 0.9990234375]}}
    else:
        layer = {"type": "attention", "mlp": None,
                 "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25, "rot": {"base": 10000.0, "dims": 8}}}
        if kind == "chunked":
            layer["mixer"]["mask"] = {"size": CHUNK}
    raw = nu.single(layer, width=32, vocab=64)
    w = nu.make_weights(raw, seed=9)
    w["embed"][:, 0:2] = 0.0
    w["embed"][NEEDLE, 0] = 8.0
    w["embed"][ASK, 1] = 8.0
    strength = 8.0 if kind == "lightning" else 4.0
    for name, column in (("k", 0), ("q", 1)):
        w["l0.mix." + name][:, 0:2] = 0.0
        for h in range(w["l0.mix." + name].shape[0] // 16):
            w["l0.mix." + name][h * 16 + AT, :] = 0.0
            w["l0.mix." + name][h * 16 + AT, column] = strength
    w["l0.mix.o"] *= 4.0            # the layer's branch outweighs the embedding's own share of the logits
    return raw, {k: v.to(torch.bfloat16).float() for k, v in w.items()}


def cut_in_pairs(requests, first_wanted, alone=3, sizes=(129, 2, 255, 31, 64, 3)):
    """Two requests side by side on two slots, in portions of changing size; each request's last ``alone`` tokens
    come one by one; logits are wanted from position ``first_wanted`` on."""
    steps = []
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
                size = 1 if left <= alone else min(sizes[(turn + index) % len(sizes)], left - alone)
                want = [i for i in range(size) if fed[rid] + i >= first_wanted]
                entries.append({"id": rid, "tokens": tokens[fed[rid]: fed[rid] + size], "want": want})
                fed[rid] += size
                if fed[rid] == len(tokens):
                    end.append(rid)
            turn += 1
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def moved_by_the_needle(raw, weights, tokens, plain_rows, row):
    """How far the plain logits of ``row`` move when the needle is taken away, as a share of their spread."""
    blind = list(tokens)
    blind[blind.index(NEEDLE)] = FILLERS + 3
    diff = pn.forward(raw, weights, blind).float()[row] - plain_rows[row]
    return float((diff - diff.mean()).pow(2).mean().sqrt() / plain_rows[row].std())


@functools.lru_cache(maxsize=None)
def chunk_case():
    """(Made once for both precisions: the plain implementation walks every key of every token.)"""
    raw, weights = planted("chunked")
    askers = [597, 599, 600, 602]           # 400 .. 599 is one chunk, 600 .. the next
    length = 603
    places = [0, 1, 199, 200, 399, 400, 401, 511, 512, 596, 598, 601]
    requests = {}
    for place in places:
        tokens = [FILLERS + t % (raw["vocab"] - FILLERS) for t in random_tokens(length, 1000, 30 + place)]
        for asker in askers:
            tokens[asker] = ASK
        tokens[place] = NEEDLE
        requests[f"n{place}"] = tokens
    plain = plain_all(raw, weights, requests)
    moved = lambda place, row: moved_by_the_needle(raw, weights, requests[f"n{place}"], plain[f"n{place}"], row)
    assert moved(400, 597) > 0.3 and moved(399, 597) < 1e-6 and moved(0, 597) < 1e-6
    assert moved(598, 599) > 0.3 and moved(598, 600) < 1e-6 and moved(596, 602) < 1e-6
    assert moved(601, 602) > 0.3 and moved(401, 599) > 0.3
    return raw, weights, requests, plain, length


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_is_seen_inside_its_chunk_and_not_outside(dtype):
    """Askers at the last tokens of a chunk (inside a prompt's portion) and at the first tokens of the next one
    (decoded alone); the needle at the chunk's first token and the one before it, at its last token, at page
    borders, at the first positions.  A key seen or lost by one token too many moves these logits by far more than
    the tolerance (checked below on the plain implementation itself)."""
    raw, weights, requests, plain, length = chunk_case()
    steps = cut_in_pairs(requests, first_wanted=597)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = nu.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == list(range(597, length)) for rid in requests)
    worst, _ = nu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0


@functools.lru_cache(maxsize=None)
def far_case(kind):
    raw, weights = planted(kind)
    length = 600
    places = [0, 1, 15, 16, 17, 63, 64, 300, 511, 512, 590]
    requests = {}
    for place in places:
        tokens = [FILLERS + t % (raw["vocab"] - FILLERS) for t in random_tokens(length, 1000, 30 + place)]
        tokens[place] = NEEDLE
        requests[f"n{place}"] = tokens + [ASK, FILLERS, ASK]
    plain = plain_all(raw, weights, requests)
    for place in (0, 300):
        for row in (length, length + 2):
            assert moved_by_the_needle(raw, weights, requests[f"n{place}"], plain[f"n{place}"], row) > 0.3
    return raw, weights, requests, plain, length


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["unchunked", "lightning"])
def test_one_key_among_hundreds_is_found_wherever_it_lies(kind, dtype):
    """The needle at the first positions, at page borders, far back; asked for inside a prompt's portion and by a
    token decoded alone, across several requests that share a pool and reuse slots.  A lost key, a key of a wrong
    page or slot, or a memory that is not carried moves these logits by far more than the tolerance."""
    raw, weights, requests, plain, length = far_case(kind)
    steps = cut_in_pairs(requests, first_wanted=length, alone=1)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = nu.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == [length, length + 1, length + 2] for rid in requests)
    worst, _ = nu.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A prompt of 150 tokens, then 250 tokens decoded one by one: chunks of 20 and of 5 tokens begin and end among
    the decoded tokens, pages are crossed and given back, memories are carried 250 times, every loop pass on its own."""
    raw = nu.SMALL_A
    weights = nu.make_weights(raw, seed=31, exact_router=True)
    requests = {"long": random_tokens(400, raw["vocab"], 7)}
    stepper = pn.Stepper(raw, weights)
    plain = {"long": torch.cat([stepper.feed([t]) for t in requests["long"]]).float()}
    steps = replay_util.tail_one_by_one(requests, tail=250)
    run_and_compare(raw, weights, requests, steps, dtype, plain, max_running=1)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
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
        engine.model.load(nu.Fixed(weights), dtype, "cuda:0")
        results = engine.generate(prompts, GenerationConfig(max_output_tokens=12))
        for prompt, result in zip(prompts, results):
            assert len(result.token_ids) == 12
            turned = replay_util.greedy_tokens_follow_plain(
                lambda tokens: pn.forward(raw, weights, tokens), prompt, result.token_ids,
                (lambda tokens: pn.forward(raw, weights, tokens, dtype=torch.bfloat16)) if dtype == "bfloat16" else None)
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
    worst, _ = nu.spread(replay_util.by_position(steps, outputs), plain)
    assert worst <= LIMIT["float32"], worst


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_norm_in_groups_adds_what_the_stream_is_owed(dtype):
    """A branch (with and without a gate), rows of a sum with a weight each, rows that join the stream once more,
    any of them or none; one group and many; only some rows handed back."""
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(2)
    for rows, hidden, groups, n_parts in ((3, 40, 5, 0), (70, 192, 2, 3), (9, 2048, 1, 4), (5, 50, 50, 2), (130, 1024, 8, 1)):
        residual = torch.randn(rows, hidden, generator=g)
        branch = torch.randn(rows, hidden, generator=g).to(dtype)
        gate = torch.randn(rows, generator=g) * 2
        parts = torch.randn(rows, max(n_parts, 1), hidden, generator=g)
        part_weight = torch.rand(rows, max(n_parts, 1), generator=g) * 2
        plus = torch.randn(rows, hidden, generator=g)
        weight = 1.0 + 0.3 * torch.randn(hidden, generator=g)
        wide_gate = torch.zeros(rows, 5).cuda()
        wide_gate[:, 2] = gate.cuda()       # (one logit per row, the rows five floats apart)
        tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=1e-2, rtol=1e-2)
        for use_branch, use_gate, use_parts, use_weight, use_plus in (
                (True, True, True, True, True), (True, False, False, False, False), (False, False, True, True, False),
                (False, False, False, False, True), (False, False, False, False, False), (True, True, True, False, False)):
            if use_parts and not n_parts:
                continue
            stream = residual.clone().cuda()
            out = ops.group_norm_add(
                stream, branch.cuda() if use_branch else None, weight.cuda(), groups, 1e-5, dtype,
                branch_gate=wide_gate[:, 2] if use_gate else None, parts=parts.cuda() if use_parts else None,
                part_weight=part_weight.cuda() if use_weight else None, plus=plus.cuda() if use_plus else None)
            want = residual.double()
            if use_branch:
                want = want + branch.double() * (torch.sigmoid(gate.double())[:, None] if use_gate else 1.0)
            if use_parts:
                want = want + (parts.double() * (part_weight.double()[:, :, None] if use_weight else 1.0)).sum(1)
            if use_plus:
                want = want + plus.double()
            assert torch.allclose(stream.double().cpu(), want, atol=2e-5)
            normed = pn.grouped_norm(want, weight.double(), groups, 1e-5)
            assert out.dtype == dtype and torch.allclose(out.double().cpu(), normed, **tol)
        picked = torch.tensor([rows - 1, 0], dtype=torch.int32)
        stream = residual.clone().cuda()
        some = ops.group_norm_add(stream, branch.cuda(), weight.cuda(), groups, 1e-5, dtype, rows=picked.cuda())
        want = pn.grouped_norm(residual.double() + branch.double(), weight.double(), groups, 1e-5)[picked.long()]
        assert some.shape == (2, hidden) and torch.allclose(some.double().cpu(), want, **tol)


@pytest.mark.parametrize("sizes", [(150, 8, 2, 2, (5, 2)), (7, 70, 0, 1, None), (33, 3, 3, 3, (3, 2)), (600, 12, 4, 4, (4, 2)),
                                   (40, 1, 5, 6, (2, 2)), (64, 250, 6, 8, (64, 3)), (19, 6, 0, 6, (3, 3))])
def test_routing_with_softmax_scores_corrections_and_groups(sizes):
    """Choice and weights against the plain router, token by token; pairs in order of their experts, and only pairs
    of experts that have weights in tiles."""
    from cie_amd.kernels import ops

    T, E, identity, top, groups = sizes
    outputs = E + identity
    g = torch.Generator().manual_seed(T)
    logits = torch.randn(T, outputs, generator=g) * 2
    correction = torch.rand(outputs, generator=g) * 0.5 - 0.35
    count, keep = groups or (1, 1)
    for scale, with_correction in ((2.5, True), (1.0, False)):
        route = ops.experts_route(logits.cuda(), top, 16, real=E, scoring="softmax",
                                  correction=correction.cuda() if with_correction else None, groups=groups,
                                  normalize=True, scale=scale)
        got_e = route.pair_expert.cpu().reshape(T, top).tolist()
        got_w = route.pair_weight.cpu().reshape(T, top).double()
        for t in range(T):
            chosen, weights = pn.router_choice(logits[t].double(), correction.double() if with_correction else torch.zeros(outputs, dtype=torch.float64),
                                               top, count, keep, scale)
            assert got_e[t] == chosen, (t, got_e[t], chosen)
            assert torch.allclose(got_w[t], weights, atol=1e-6, rtol=1e-5)
        flat = route.pair_expert.cpu().long()
        n = int(route.n_tiles.cpu())
        assert n <= route.max_tiles and int(route.tile_count.cpu()[:n].sum()) == int((flat < E).sum())
        order = route.sorted.cpu().long()[: int((flat < E).sum())]
        assert bool((flat[order] < E).all()) and bool((flat[order].diff() >= 0).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_whose_weight_waits_for_the_sum_and_experts_that_hand_rows_on(dtype):
    from cie_amd.kernels import ops

    T, E, identity, top, width, ff = 90, 5, 2, 3, 64, 40
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, width, generator=g).to(dtype)
    logits = torch.randn(T, E + identity, generator=g) * 2
    w = {(e, n): (torch.randn(*s, generator=g) * 1.5 / s[1] ** 0.5).to(dtype).float()
         for e in range(E) for n, s in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff)))}
    gate_up = torch.stack([torch.cat([w[e, "gate"], w[e, "up"]]) for e in range(E)]).to(dtype).cuda()
    down = torch.stack([w[e, "down"] for e in range(E)]).to(dtype).cuda()
    mfma = dtype == torch.bfloat16
    for tile_rows in ((16, 32, 64, 128) if mfma else (16,)):
        route = ops.experts_route(logits.cuda(), top, tile_rows, real=E, scoring="softmax", normalize=True, scale=2.0)
        parts = ops.experts_forward(x.cuda(), route, gate_up, down, float("inf"), 1.0, 0.0, mfma=mfma, weight_input=False).cpu().double()
        chosen = route.pair_expert.cpu().reshape(T, top).tolist()
        tol = 2e-5 if dtype == torch.float32 else 3e-2
        for t in range(T):
            for j, e in enumerate(chosen[t]):
                h = x[t].double()
                want = h if e >= E else pn.gated_expert(h, w[e, "gate"].double(), w[e, "up"].double(), w[e, "down"].double())
                assert torch.allclose(parts[t, j], want, atol=tol, rtol=tol), (t, j, e, tile_rows)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_bounded_unit_with_other_constants(dtype):
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(5)
    gate_up = (torch.randn(11, 2 * 37, generator=g) * 3).to(dtype)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    for limit, alpha, offset in ((1.0, 1.702, 1.0), (0.25, 1.702, 1.0), (float("inf"), 1.0, 0.0), (2.0, 0.5, -1.0)):
        got = ops.clamped_glu(gate_up.cuda(), limit, alpha, offset).double().cpu()
        gate, up = gate_up[:, :37].double().clamp(max=limit), gate_up[:, 37:].double().clamp(-limit, limit)
        assert torch.allclose(got, gate * torch.sigmoid(alpha * gate) * (up + offset), atol=tol, rtol=tol)
