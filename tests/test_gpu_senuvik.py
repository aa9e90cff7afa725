"""GPU: the Senuvik decoder in the engine against the plain implementation (tests/plain_senuvik.py): every mechanism
alone, every way of cutting and batching the same requests, reused pages and slots, keys at the window's edges, among
the kept first tokens and far back, long decoding, other sizes, greedy generation through the engine's own entry
point, and the new kernels alone."""

from __future__ import annotations

import copy
import functools
import random

import numpy as np
import pytest
import torch

import plain_senuvik as ps
import replay_util
import senuvik_util as su
from conftest import random_tokens

pytestmark = pytest.mark.gpu

# a row's error is the root mean square of the difference of its logits, mean taken off, as a share of the
# logits' own spread.  float32: sums in another order; this is the sharp test of cache, state and batching.
# bfloat16: activations rounded to 8 bits between kernels, with these bold weights a few per cent at the worst row.
LIMIT = {"float32": 2e-5, "bfloat16": 8e-2}
RMS_LIMIT = {"float32": 1e-5, "bfloat16": 3e-2}


def plain_all(raw, weights, requests):
    return {rid: ps.forward(raw, weights, tokens).float() for rid, tokens in requests.items()}


def run_and_compare(raw, weights, requests, steps, dtype, plain, page_size=16, max_running=4, limit=None, graph_decode=False):
    pool = max(replay_util.max_live_tokens(steps, page=page_size), page_size)
    runner = su.make_runner(raw, weights, dtype, pool, page_size, max_running, graph_decode=graph_decode)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    for rid in requests:
        assert rid in rows, f"{rid}: no logits"
    worst, rms = su.spread(rows, plain)
    assert worst <= (limit or LIMIT[dtype]) and rms <= RMS_LIMIT[dtype], (dtype, worst, rms)
    assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0
    return rows


TINY = {"heads": 1, "vdim": 4, "state": 2, "groups": 1, "conv": 2, "norm_groups": 1}
ROT = {"base": 200.0, "dims": 8, "scaling": {"factor": 4.0}}
WRITER = {"type": "attention", "mlp": None,
          "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.4, "mask": {"size": 7, "keep_first": 2}, "rot": ROT}}

MECHANISMS = {
    # a window that ends inside pages, kept first tokens, two query heads a key head, a rotation over half of the head
    "attention": WRITER,
    # a window of one token beside five kept ones; one key head for all; every number turns
    "attention_alone_in_its_window": {"type": "attention", "mlp": None,
                                      "mixer": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 24, "scale": 0.6,
                                                "mask": {"size": 1, "keep_first": 5}, "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 1.5}}}},
    # more kept first tokens than a page holds, no key is ever lost before position 40
    "attention_many_kept": {"type": "attention", "mlp": None,
                            "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 24, "scale": 0.3,
                                      "mask": {"size": 3, "keep_first": 37}, "rot": {"base": 30.0, "dims": 6, "scaling": {"factor": 2.0}}}},
    # head sizes of the matrix-core kernels; kept first tokens that fill blocks of 32 keys and more
    "attention_heads_of_64": {"type": "attention", "mlp": None,
                              "mixer": {"heads": 6, "kv_heads": 3, "dim": 64, "vdim": 64, "scale": 0.15,
                                        "mask": {"size": 9, "keep_first": 3}, "rot": {"base": 300000.0, "dims": 32, "scaling": {"factor": 4.0}}}},
    "attention_heads_of_128_and_64": {"type": "attention", "mlp": None,
                                      "mixer": {"heads": 4, "kv_heads": 2, "dim": 128, "vdim": 64, "scale": 0.1,
                                                "mask": {"size": 5, "keep_first": 2}, "rot": {"base": 5000.0, "dims": 48, "scaling": {"factor": 3.0}}}},
    "space": {"type": "mamba2", "mlp": None,
              "mixer": {"heads": 4, "vdim": 8, "state": 12, "groups": 2, "conv": 4, "norm_groups": 2}},
    "space_one_of_each": {"type": "mamba2", "mlp": None,
                          "mixer": {"heads": 1, "vdim": 40, "state": 5, "groups": 1, "conv": 1, "norm_groups": 1}},
    # a memory of more rows than one thread keeps, every head a group of its own, as many norm groups as heads
    "space_tall": {"type": "mamba2", "mlp": None,
                   "mixer": {"heads": 3, "vdim": 16, "state": 136, "groups": 3, "conv": 3, "norm_groups": 3}},
    "space_wide": {"type": "mamba2", "mlp": None,
                   "mixer": {"heads": 2, "vdim": 72, "state": 64, "groups": 1, "conv": 5, "norm_groups": 4}},
    "pair": {"type": "parallel", "mlp": None,
             "mixer": {"left": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.35, "softcap": 5.0,
                                "rot": {"base": 1000.0, "dims": 8, "scaling": su.YARN}},
                       "right": {"heads": 2, "dim": 12}, "left_scale": 0.7, "right_scale": 0.4}},
    # every number of the left heads turns, no stretch; right heads of 64; one side counts nothing
    "pair_heads_of_64": {"type": "parallel", "mlp": None,
                         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.12, "softcap": 40.0,
                                            "rot": {"base": 300000.0, "dims": 64}},
                                   "right": {"heads": 2, "dim": 64}, "left_scale": 1.0, "right_scale": 1.5}},
    "pair_left_alone": {"type": "parallel", "mlp": None,
                        "mixer": {"left": {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 16, "scale": 0.5, "softcap": 2.0,
                                           "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 8.0, "fast": 4.0, "original": 16, "slow": 0.5}}},
                                  "right": {"heads": 1, "dim": 4}, "left_scale": 2.0, "right_scale": 0.0}},
    "pair_right_alone": {"type": "parallel", "mlp": None,
                         "mixer": {"left": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.5, "softcap": 2.0,
                                            "rot": {"base": 100.0, "dims": 8}},
                                   "right": {"heads": 5, "dim": 24}, "left_scale": 0.0, "right_scale": 1.0}},
    "dense": {"type": "mamba2", "mixer": TINY, "mlp": {"kind": "dense", "ff": 44}},
    "experts": {"type": "mamba2", "mixer": TINY, "mlp": su.MOE_A},
    "experts_without_shared": {"type": "mamba2", "mixer": TINY,
                               "mlp": {"kind": "moe", "router": {"experts": 5, "top": 2}, "expert": {"ff": 40}}},
    "experts_all_chosen": {"type": "mamba2", "mixer": TINY,
                           "mlp": {"kind": "moe", "router": {"experts": 4, "top": 4}, "expert": {"ff": 16}, "shared": {"ff": 8}}},
    "experts_one_chosen": {"type": "mamba2", "mixer": TINY,
                           "mlp": {"kind": "moe", "router": {"experts": 9, "top": 1}, "expert": {"ff": 16}, "shared": {"ff": 40}}},
}
# a layer without keys and values of its own behind the layer it reads: a longer window, a shorter one, other kept tokens
READERS = {
    "reader_longer_window": {"size": 19, "keep_first": 0},
    "reader_shorter_window": {"size": 2, "keep_first": 2},
    "reader_more_kept": {"size": 7, "keep_first": 11},
}


def mechanism(name: str) -> dict:
    if name in READERS:
        reader = copy.deepcopy(WRITER)
        reader["mixer"].update(kv_from=0, mask=READERS[name], scale=0.3)
        reader["mlp"] = {"kind": "dense", "ff": 24}
        return su.single(reader, before=copy.deepcopy(WRITER))
    return su.single(copy.deepcopy(MECHANISMS[name]))


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS) + sorted(READERS))
def test_a_mechanism_alone(name, dtype):
    """One layer of one kind: whole prompts, then the same tokens in portions down to two tokens and one by one
    (across pages and windows), requests side by side.  Routers read the whole stream in float32 and markers in
    bfloat16, where a near-tie could turn."""
    raw = mechanism(name)
    weights = su.make_weights(raw, seed=3, exact_router=dtype == "bfloat16")
    requests = {"a": random_tokens(75, raw["vocab"], 1), "b": random_tokens(21, raw["vocab"], 2), "c": [7]}
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
    for index, (name, raw) in enumerate(su.SMALL.items()):
        weights = su.make_weights(raw, seed=20 + index, exact_router=True)
        requests = {f"{name}{i}": random_tokens(n, raw["vocab"], seed=50 + i) for i, n in enumerate(LENGTHS[name])}
        out[name] = (raw, weights, requests, plain_all(raw, weights, requests))
    return out


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("name", sorted(su.SMALL))
def test_logits_do_not_depend_on_cutting_or_batching(models, name, schedule, dtype):
    """Prefill against token-by-token decoding, portions of several sizes, unequal requests in one batch against
    each alone; more requests than slots take turns, and the pool is no larger than the schedule's peak."""
    raw, weights, requests, plain = models[name]
    run_and_compare(raw, weights, requests, SCHEDULES[schedule](requests), dtype, plain)


def test_routers_that_read_the_whole_stream(models):
    """Float32, weights without markers: routers on ordinary rows."""
    for name, (raw, _, requests, _) in models.items():
        weights = su.make_weights(raw, seed=40, rank=5)
        plain = plain_all(raw, weights, requests)
        run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=2), "float32", plain, max_running=3)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(su.SMALL))
def test_captured_steps_give_the_same_logits(models, name, dtype):
    """Steps of single tokens replay captured graphs (and short mixed steps theirs, from the second time a shape
    comes), with uncaptured steps between the replays: every replay is checked against the plain logits, and
    memories move on once per token although a capture runs the kernels on rows of padding."""
    raw, weights, requests, plain = models[name]
    steps = replay_util.fixed_portions(requests, portion=8, live=3, decode_tail=14)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = su.make_runner(raw, weights, dtype, pool, 16, 4, graph_decode=True)
    assert runner.graphs is not None, "the model's parts all say that they may be captured"
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    worst, rms = su.spread(rows, plain)
    assert runner.graph_replays >= 10 and runner.mixed_graph_replays > 0, (runner.graph_replays, runner.mixed_graph_replays)
    assert worst <= LIMIT[dtype] and rms <= RMS_LIMIT[dtype], (worst, rms)


@pytest.mark.parametrize("page_size", [4, 64])
def test_other_page_sizes(models, page_size):
    raw, weights, requests, plain = models["A"]
    run_and_compare(raw, weights, requests, replay_util.mixed(requests, live=3, seed=5), "float32", plain,
                    page_size=page_size, max_running=3)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(su.SMALL))
def test_random_traces_reuse_pages_and_slots(models, name, dtype):
    """Random cuts (one token, two, up to a page's edge, one past it) of ten requests on three slots: every slot
    and page is handed out again, and a memory that a new request found uncleared would show at its first token."""
    raw, weights, _, _ = models[name]
    rng = random.Random(4)
    requests, steps = replay_util.random_trace(rng, [3, 40, 17, 1, 33, 64, 2, 18, 49, 31], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    pool = max(replay_util.max_live_tokens(steps, page=16), 16)
    runner = su.make_runner(raw, weights, dtype, pool, 16, 3)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert set(rows) <= set(requests) and rows
    worst, _ = su.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


def random_configuration(rng: random.Random) -> dict:
    """A model whose every size, count, constant and layer order is drawn: widths and heads that are and are not
    multiples of 8 or 64, windows shorter than a page and longer than any request, readers of earlier layers' keys."""
    width = rng.choice([24, 40, 50, 64, 96, 136])
    layers: list[dict] = []
    writers: list[int] = []

    def rotation(dim: int, stretched: bool) -> dict:
        rot = {"base": rng.choice([10.0, 1000.0, 2.0e5]), "dims": rng.choice([d for d in (2, 4, 8, 16, 64, 96, 128) if d <= dim])}
        if stretched and rng.random() < 0.7:
            rot["scaling"] = {"factor": rng.choice([2.0, 8.0]), "original": rng.choice([16, 64, 2048]),
                              "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([0.5, 1.0])}
        elif not stretched:
            rot["scaling"] = {"factor": rng.choice([1.0, 2.0, 4.0])}
        return rot

    def attention_sizes() -> dict:
        kv_heads, dim = rng.choice([1, 2, 3]), rng.choice([8, 16, 24, 64, 96, 128])
        return {"heads": kv_heads * rng.choice([1, 2, 6]), "kv_heads": kv_heads, "dim": dim,
                "vdim": rng.choice([8, 24, 64, 128]), "scale": rng.choice([0.5, 1.0, 2.0]) * dim ** -0.5}

    for index in range(rng.randint(2, 6)):
        kind = rng.choice(["attention", "mamba2", "parallel"])
        if kind == "attention":
            mask = {"size": rng.choice([1, 3, 16, 17, 31, 45, 64, 500]), "keep_first": rng.choice([0, 1, 4, 18, 33, 70])}
            if writers and rng.random() < 0.5:
                source = rng.choice(writers)
                mixer = copy.deepcopy(layers[source]["mixer"])
                mixer.update(kv_from=source, mask=mask, scale=mixer["scale"] * rng.choice([0.5, 1.0]))
            else:
                mixer = attention_sizes()
                mixer.update(mask=mask, rot=rotation(mixer["dim"], False))
                writers.append(index)
        elif kind == "mamba2":
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2, 4])
            mixer = {"heads": heads, "vdim": rng.choice([4, 8, 32, 64, 72]), "state": rng.choice([1, 5, 16, 56, 64, 128, 136]),
                     "groups": groups, "conv": rng.choice([1, 2, 4, 7]), "norm_groups": rng.choice([1, heads])}
        else:
            left = attention_sizes()
            left.update(softcap=rng.choice([2.0, 30.0, 80.0]), rot=rotation(left["dim"], True))
            mixer = {"left": left, "right": {"heads": rng.choice([1, 2, 4, 5]), "dim": rng.choice([4, 12, 40, 64, 72])},
                     "left_scale": rng.choice([0.5, 0.6, 1.0]), "right_scale": rng.choice([0.5, 1.0, 1.5])}
        draw = rng.random()
        if draw < 0.15:
            mlp = None
        elif draw < 0.5:
            mlp = {"kind": "dense", "ff": rng.choice([24, 52, 100])}
        else:
            experts = rng.choice([1, 2, 3, 5, 16])
            mlp = {"kind": "moe", "expert": {"ff": rng.choice([8, 20, 48])}, "router": {"experts": experts, "top": rng.randint(1, min(experts, 4))}}
            if rng.random() < 0.7:
                mlp["shared"] = {"ff": rng.choice([8, 28])}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Senuvik", "vocab": rng.choice([70, 130, 300]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_and_traces(seed):
    """Models that nobody chose, each under a random trace of six requests on three slots, in both precisions."""
    rng = random.Random(2000 + seed)
    raw = random_configuration(rng)
    weights = su.make_weights(raw, seed=seed, exact_router=True, rank=rng.choice([1, 4, 16, 33]))
    requests, steps = replay_util.random_trace(rng, [rng.choice([1, 2, 9, 33, 48, 90]) for _ in range(6)], raw["vocab"], 16, live_most=3)
    plain = plain_all(raw, weights, requests)
    for dtype in ("float32", "bfloat16"):
        runner = su.make_runner(raw, weights, dtype, max(replay_util.max_live_tokens(steps, page=16), 16), 16, 3)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        assert rows
        worst, rms = su.spread(rows, plain)
        if dtype == "float32":
            # (six layers deep, float32 sums in another order than the yardstick's float64 reach 2.5e-5 at the worst row)
            assert worst <= 2.5 * LIMIT[dtype] and rms <= RMS_LIMIT[dtype], (dtype, worst, rms, raw)
        else:
            # up to six layers whose branches are all brought to the same size before they are added: what bfloat16
            # costs grows with the depth, evenly over the layers, and differs from model to model.  It is measured,
            # not assumed: over all rows the engine has to be closer to the float32 logits than the plain
            # implementation run in bfloat16 throughout is.  The worst row may lie further out than the plain one's: a
            # sequence's first token leaves a time-mixing head's read-out a multiple of one vector, the norm behind it
            # divides by that multiple, and where it is small any rounding in front of it shows in full.
            rough = {rid: ps.forward(raw, weights, tokens, dtype=torch.bfloat16).float() for rid, tokens in requests.items()}
            mine = [float((torch.from_numpy(rows[rid][pos]) - plain[rid][pos]).pow(2).mean()) for rid in rows for pos in rows[rid]]
            theirs = [float((rough[rid][pos] - plain[rid][pos]).pow(2).mean()) for rid in rows for pos in rows[rid]]
            assert sum(mine) <= sum(theirs) and max(mine) <= 9.0 * max(theirs), (sum(mine), sum(theirs), max(mine), max(theirs), raw)
        assert runner.cache.stats().slots_used == 0 and runner.cache.stats().pages_used == 0


# ---------------------------------------------------------------- keys and memories that random weights would hide
NEEDLE, ASK, FILLERS = 1, 2, 40  # token ids: the one to be found, the one that looks for it, the first of the rest
AT = 12                          # the head's number that carries the mark: one that does not turn
WINDOW, KEPT = 100, 37


def planted(kind: str):
    """A single layer whose weights are changed by hand so that one score stands out: the token ASK looks, through a
    query number that only it has, for a key number that only the token NEEDLE has, wherever that lies."""
    if kind == "space":
        layer = {"type": "mamba2", "mlp": None,
                 "mixer": {"heads": 2, "vdim": 16, "state": 16, "groups": 1, "conv": 1, "norm_groups": 1}}
    elif kind == "time":
        layer = {"type": "parallel", "mlp": None,
                 "mixer": {"left": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.3, "softcap": 20.0,
                                    "rot": {"base": 100.0, "dims": 8}},
                           "right": {"heads": 2, "dim": 16}, "left_scale": 0.0, "right_scale": 1.0}}
    else:
        layer = {"type": "attention", "mlp": None,
                 "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.5,
                           "mask": {"size": WINDOW if kind == "window" else 100000, "keep_first": KEPT if kind == "window" else 0},
                           "rot": {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0}}}}
    raw = su.single(layer, width=32, vocab=64)
    w = su.make_weights(raw, seed=9)
    w["embed"][:, 0:2] = 0.0
    w["embed"][NEEDLE, 0] = 8.0
    w["embed"][ASK, 1] = 8.0
    if kind == "space":
        # B reads the needle's mark, C the asker's; the steps are small and the decays close to one
        inner, n = 32, 16
        rows = w["l0.mix.in"]
        rows[2 * inner: 2 * inner + 2 * n, 0:2] = 0.0   # (B and C of the other rows do not see the marks)
        rows[2 * inner: 2 * inner + 2 * n] *= 0.25
        rows[2 * inner + 3, :] = 0.0
        rows[2 * inner + n + 3, :] = 0.0
        rows[2 * inner + 3, 0] = 12.0         # B, row 3
        rows[2 * inner + n + 3, 1] = 12.0     # C, row 3
        w["l0.mix.conv"][:] = 1.0             # (one tap: the convolution hands its input on)
        w["l0.mix.conv.b"][:] = 0.0
        w["l0.mix.dt_bias"][:] = torch.tensor([-6.0, -6.5])
        w["l0.mix.A_log"][:] = torch.tensor([-2.0, -1.5])
    elif kind == "time":
        for name, column in (("k", 0), ("r", 1)):
            w["l0.mix.right." + name][:, 0:2] = 0.0
            for h in range(2):
                w["l0.mix.right." + name][h * 16 + 3, :] = 0.0
                w["l0.mix.right." + name][h * 16 + 3, column] = 6.0
        for s in "rkvgw":
            w["l0.mix.right.mu." + s][:] = 0.0                # every mix is the token's own input
        w["l0.mix.right.w0"][:] = -6.5                        # decays of 0.9985 a token
        w["l0.mix.right.w2"][:] = 0.0
    else:
        for name, column in (("k", 0), ("q", 1)):
            w["l0.mix." + name][:, 0:2] = 0.0
            w["l0.mix." + name + ".b"][:] = 0.0
            w["l0.mix." + name + ".norm"][:] = 1.0
            for h in range(w["l0.mix." + name].shape[0] // 16):
                w["l0.mix." + name][h * 16 + AT, :] = 0.0
                w["l0.mix." + name][h * 16 + AT, column] = 4.0
        w["l0.mix.sink"][:] = 0.0
    w["l0.ls1"] *= 4.0                # the layer's branch outweighs the embedding's own share of the logits
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
    diff = ps.forward(raw, weights, blind).float()[row] - plain_rows[row]
    return float((diff - diff.mean()).pow(2).mean().sqrt() / plain_rows[row].std())


@functools.lru_cache(maxsize=None)
def window_case():
    """(Made once for both precisions: the plain implementation walks every key of every token.)"""
    raw, weights = planted("window")
    askers = [597, 599, 600, 602]           # the window of 597 starts at 498, that of 602 at 503
    length = 603
    places = [0, 1, 31, 32, KEPT - 1, KEPT, KEPT + 1, 63, 64, 300, 497, 498, 500, 502, 503, 596, 601]
    requests = {}
    for place in places:
        tokens = [FILLERS + t % (raw["vocab"] - FILLERS) for t in random_tokens(length, 1000, 30 + place)]
        for asker in askers:
            tokens[asker] = ASK
        tokens[place] = NEEDLE
        requests[f"n{place}"] = tokens
    plain = plain_all(raw, weights, requests)
    moved = lambda place, row: moved_by_the_needle(raw, weights, requests[f"n{place}"], plain[f"n{place}"], row)
    assert moved(498, 597) > 0.3 and moved(497, 597) < 1e-6 and moved(498, 599) < 1e-6 and moved(500, 599) > 0.3
    assert moved(502, 602) < 1e-6 and moved(503, 602) > 0.3 and moved(601, 602) > 0.3 and moved(601, 600) < 1e-6
    assert moved(KEPT - 1, 597) > 0.3 and moved(KEPT, 597) < 1e-6 and moved(0, 602) > 0.3 and moved(300, 602) < 1e-6
    return raw, weights, requests, plain, length


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_is_seen_inside_the_window_and_among_the_kept_first_tokens_and_nowhere_else(dtype):
    """Askers inside a prompt's portion and decoded alone; the needle at the window's first token and the one before
    it, at its last token, at the last kept token and the first one that is not kept, at page borders and at the first
    positions.  A key seen or lost by one token too many moves these logits by far more than the tolerance (checked
    on the plain implementation itself)."""
    raw, weights, requests, plain, length = window_case()
    steps = cut_in_pairs(requests, first_wanted=597)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = su.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == list(range(597, length)) for rid in requests)
    worst, _ = su.spread(rows, plain)
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
            assert moved_by_the_needle(raw, weights, requests[f"n{place}"], plain[f"n{place}"], row) > 0.3, (kind, place, row)
    return raw, weights, requests, plain, length


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["all_keys", "space", "time"])
def test_one_token_among_hundreds_is_found_wherever_it_lies(kind, dtype):
    """The needle at the first positions, at page borders, far back; asked for inside a prompt's portion and by a
    token decoded alone, across several requests that share a pool and reuse slots.  A lost key, a key of a wrong
    page or slot, or a memory that is not carried moves these logits by far more than the tolerance."""
    raw, weights, requests, plain, length = far_case(kind)
    steps = cut_in_pairs(requests, first_wanted=length, alone=1)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = su.make_runner(raw, weights, dtype, pool, 16, 2)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert all(sorted(rows[rid]) == [length, length + 1, length + 2] for rid in requests)
    worst, _ = su.spread(rows, plain)
    assert worst <= LIMIT[dtype], worst


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mask", [(300, 70), (260, 0), (130, 200), (512, 31)])
def test_long_windows_behind_kept_tokens(mask, dtype):
    """Windows long enough for the matrix-core kernel to cut a decoded token's keys into shares, with kept first
    tokens that fill blocks of keys, end inside one, or outnumber the window: prompts of 700 tokens in one portion and
    in several, then forty tokens decoded one by one, two requests side by side."""
    size, keep = mask
    layer = {"type": "attention", "mlp": None,
             "mixer": {"heads": 4, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.2, "mask": {"size": size, "keep_first": keep},
                       "rot": {"base": 10000.0, "dims": 16, "scaling": {"factor": 2.0}}}}
    raw = su.single(layer, width=64, vocab=80)
    weights = su.make_weights(raw, seed=12)
    requests = {"a": random_tokens(700, raw["vocab"], 3), "b": random_tokens(611, raw["vocab"], 4)}
    plain = plain_all(raw, weights, requests)
    run_and_compare(raw, weights, requests, replay_util.tail_one_by_one(requests, tail=40), dtype, plain)
    steps = cut_in_pairs(requests, first_wanted=0, alone=40, sizes=(129, 2, 255, 31, 64, 3))
    run_and_compare(raw, weights, requests, steps, dtype, plain, max_running=2)


@pytest.mark.filterwarnings("ignore:bfloat16 attention")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A prompt of 150 tokens, then 250 tokens decoded one by one: windows pass over decoded tokens, pages are
    crossed and given back while the first ones stay, memories and the convolution's inputs are carried 250 times."""
    raw = su.SMALL_A
    weights = su.make_weights(raw, seed=31, exact_router=True)
    requests = {"long": random_tokens(400, raw["vocab"], 7)}
    plain = plain_all(raw, weights, requests)
    steps = replay_util.tail_one_by_one(requests, tail=250)
    # one of the 400 rows is ill-conditioned (a read-out of the state-space layer that nearly cancels: ten times the
    # error of every other row, the same whether the row is decoded alone or lies in a whole prompt); the root mean
    # square over the rows keeps its limit
    decoded = run_and_compare(raw, weights, requests, steps, dtype, plain, max_running=1, limit=3 * LIMIT[dtype])
    whole = run_and_compare(raw, weights, requests, replay_util.whole(requests), dtype, plain, max_running=1, limit=3 * LIMIT[dtype])
    apart = max(float(np.abs(decoded["long"][p] - whole["long"][p]).max()) for p in whole["long"])
    assert apart <= (2e-4 if dtype == "float32" else 0.5), apart


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
        engine.model.load(su.Fixed(weights), dtype, "cuda:0")
        results = engine.generate(prompts, GenerationConfig(max_output_tokens=12))
        for prompt, result in zip(prompts, results):
            assert len(result.token_ids) == 12
            turned = replay_util.greedy_tokens_follow_plain(
                lambda tokens: ps.forward(raw, weights, tokens), prompt, result.token_ids,
                (lambda tokens: ps.forward(raw, weights, tokens, dtype=torch.bfloat16)) if dtype == "bfloat16" else None)
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
    worst, _ = su.spread(replay_util.by_position(steps, outputs), plain)
    assert worst <= LIMIT["float32"], worst


# ---------------------------------------------------------------- kernels alone
def _meta(lengths):
    starts = [0]
    for n in lengths:
        starts.append(starts[-1] + n)
    seq_of_token = [s for s, n in enumerate(lengths) for _ in range(n)]
    as_int = lambda values: torch.tensor(values, dtype=torch.int32, device="cuda")
    return as_int(starts), as_int(seq_of_token)


@pytest.mark.parametrize("shape", [(2, 5, 3, 1, False), (4, 40, 24, 2, False), (3, 136, 16, 1, False), (2, 64, 72, 2, False),
                                   (2, 12, 12, 1, True), (4, 40, 40, 1, True), (1, 64, 64, 1, True), (3, 1, 9, 3, False),
                                   (2, 300, 8, 1, True)])
def test_the_memory_walk_against_a_loop(shape):
    """Both forms of the walk (a decay per head with the read-out behind the update, a decay per row with the
    read-out in front of it and a bonus) at sizes on both sides of every tile, sequences of unequal length from
    states that earlier steps left, in slots that are not in order."""
    from cie_amd.kernels import ops

    heads, rows, cols, per_group, time_form = shape
    g = torch.Generator().manual_seed(rows * 7 + cols)
    lengths = [1, 37, 2, 19] if rows < 200 else [1, 70, 2, 33]
    slots = [3, 0, 4, 1]
    tokens = sum(lengths)
    q_start_loc, _ = _meta(lengths)
    groups = heads // per_group
    decay = torch.rand(tokens, heads * rows if time_form else heads, generator=g) * 0.5 + 0.5
    in_rows = torch.randn(tokens, groups * rows, generator=g)
    out_rows = torch.randn(tokens, groups * rows, generator=g)
    values = torch.randn(tokens, heads * cols, generator=g)
    scale = None if time_form else torch.rand(tokens, heads, generator=g)
    skip = None if time_form else torch.randn(heads, generator=g)
    bonus = torch.randn(heads, rows, generator=g) if time_form else None
    state = torch.randn(6, heads, rows, cols, generator=g)
    want_state = state.double().clone()
    want = torch.zeros(tokens, heads * cols, dtype=torch.float64)
    first = 0
    for length, slot in zip(lengths, slots):
        for t in range(first, first + length):
            for h in range(heads):
                grp = h // per_group
                S = want_state[slot, h]
                a = in_rows[t, grp * rows:(grp + 1) * rows].double()
                o = out_rows[t, grp * rows:(grp + 1) * rows].double()
                v = values[t, h * cols:(h + 1) * cols].double()
                if time_form:
                    d = decay[t, h * rows:(h + 1) * rows].double()
                    want[t, h * cols:(h + 1) * cols] = (S + torch.outer(bonus[h].double() * a, v)).t() @ o
                    want_state[slot, h] = d[:, None] * S + torch.outer(a, v)
                else:
                    S = float(decay[t, h]) * S + torch.outer(a, v * float(scale[t, h]))
                    want_state[slot, h] = S
                    want[t, h * cols:(h + 1) * cols] = S.t() @ o + float(skip[h]) * v
        first += length
    cuda = lambda t: None if t is None else t.cuda()
    state_gpu = state.cuda()
    # (the row operands as views of wider rows, as the layers hand them over)
    wide = torch.cat([in_rows, out_rows, values], dim=1).cuda()
    n = groups * rows
    got = ops.memory_walk(cuda(decay), wide[:, :n], wide[:, n:2 * n], wide[:, 2 * n:], state_gpu,
                          torch.tensor(slots, dtype=torch.int32, device="cuda"), q_start_loc, len(lengths), heads, rows, cols,
                          heads_per_group=per_group, bonus=cuda(bonus), value_scale=cuda(scale), skip=cuda(skip),
                          read_first=time_form)
    assert torch.allclose(got.double().cpu(), want, rtol=1e-4, atol=1e-4)
    assert torch.allclose(state_gpu.double().cpu(), want_state, rtol=1e-4, atol=1e-4)
    untouched = [s for s in range(6) if s not in slots]
    assert torch.equal(state_gpu[untouched].cpu(), state[untouched])
    if not time_form:
        # the same in blocks of 32 tokens on the matrix cores (sequences of 1, 37, 2 and 19 tokens: whole blocks, rests)
        state_gpu = state.cuda()
        got = ops.memory_walk(cuda(decay), wide[:, :n], wide[:, n:2 * n], wide[:, 2 * n:], state_gpu,
                              torch.tensor(slots, dtype=torch.int32, device="cuda"), q_start_loc, len(lengths), heads, rows,
                              cols, heads_per_group=per_group, value_scale=cuda(scale), skip=cuda(skip),
                              log_decay=torch.log(decay).cuda(), blocks=True)
        assert torch.allclose(got.double().cpu(), want, rtol=1e-4, atol=1e-4)
        assert torch.allclose(state_gpu.double().cpu(), want_state, rtol=1e-4, atol=1e-4)
        assert torch.equal(state_gpu[untouched].cpu(), state[untouched])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_norm_on_a_branch_adds_gates_weighs_and_norms_again(dtype):
    """A branch with a gate, a second branch with scales, rows of a sum with weights, any of them; the stream's norm
    under a second weight in the same kernel."""
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(5)
    norm = lambda x, w: x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    for rows, hidden, n_parts in ((3, 40, 0), (70, 192, 3), (9, 2048, 4), (130, 50, 1)):
        residual = torch.randn(rows, hidden, generator=g)
        first = torch.randn(rows, hidden, generator=g).to(dtype)
        second = torch.randn(rows, hidden, generator=g).to(dtype)
        gate = torch.randn(rows, generator=g) * 2
        parts = torch.randn(rows, max(n_parts, 1), hidden, generator=g)
        part_weight = torch.rand(rows, max(n_parts, 1), generator=g) * 2
        weight = 1.0 + 0.3 * torch.randn(hidden, generator=g)
        after = 1.0 + 0.3 * torch.randn(hidden, generator=g)
        wide_gate = torch.zeros(rows, 8).cuda()
        wide_gate[:, 0] = gate.cuda()
        for use_first, use_gate, use_second, use_parts, use_weight, use_after in (
                (True, True, False, True, True, True), (True, False, True, False, False, True), (False, False, False, True, False, False),
                (True, False, False, False, False, False), (True, True, True, True, True, False)):
            if use_parts and not n_parts:
                continue
            stream = residual.clone().cuda()
            got = ops.branch_norm_add(
                stream, first.cuda() if use_first else None, weight.cuda(), 1e-5, dtype, want_rows=False,
                parts=parts.cuda() if use_parts else None, part_weight=part_weight.cuda() if use_weight else None,
                branch_gate=wide_gate[:, 0] if use_gate else None, branch2=second.cuda() if use_second else None,
                scales=(0.6, 1.5), next_weight=after.cuda() if use_after else None)
            y = torch.zeros(rows, hidden, dtype=torch.float64)
            if use_first:
                y = y + 0.6 * first.double() * (torch.sigmoid(gate.double())[:, None] if use_gate else 1.0)
            if use_second:
                y = y + 1.5 * second.double()
            if use_parts:
                y = y + (parts.double() * (part_weight.double()[:, :, None] if use_weight else 1.0)).sum(1)
            want = residual.double() + norm(y, weight.double())
            assert torch.allclose(stream.double().cpu(), want, atol=3e-5, rtol=1e-5)
            if use_after:
                assert got[0] is None and got[1].dtype == dtype
                assert torch.allclose(got[1].double().cpu(), norm(want, after.double()), **tol)
            else:
                assert got is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_norm_of_a_read_out_with_its_gate_on_either_side(dtype):
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(6)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    for rows, width, groups in ((3, 40, 5), (70, 192, 2), (9, 2304, 1), (5, 50, 50), (17, 1088, 17)):
        y = torch.randn(rows, width, generator=g)
        wide = torch.randn(rows, width + 24, generator=g).to(dtype)
        weight = 1.0 + 0.3 * torch.randn(width, generator=g)
        gate = wide[:, 8: 8 + width]
        for first in (True, False):
            got = ops.gated_group_norm(y.cuda(), wide.cuda()[:, 8: 8 + width], weight.cuda(), groups, 1e-5, dtype, gate_first=first)
            x = y.double() * torch.nn.functional.silu(gate.double()) if first else y.double()
            x = x.reshape(rows, groups, -1)
            x = (x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)).reshape(rows, width) * weight.double()
            if not first:
                x = x * torch.nn.functional.silu(gate.double())
            assert got.dtype == dtype and torch.allclose(got.double().cpu(), x, **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_gated_unit_with_the_tanh_form_of_gelu(dtype):
    from cie_amd.config.senuvik import GELU_ALPHA, GELU_CUBIC
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(7)
    rows = (torch.randn(33, 2 * 72, generator=g) * 3).to(dtype)
    got = ops.clamped_glu(rows.cuda(), float("inf"), GELU_ALPHA, 0.0, GELU_CUBIC)
    want = torch.nn.functional.gelu(rows[:, :72].double(), approximate="tanh") * rows[:, 72:].double()
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    assert torch.allclose(got.double().cpu(), want, **tol)


def test_token_shift_decays_and_the_convolution_carry_their_state():
    """The mixes of a token with the one before it, the decays from the two small products, and the causal
    convolution with its activation: a step's first token takes what the step before left, in its own slot."""
    from cie_amd.kernels import ops

    g = torch.Generator().manual_seed(8)
    width, channels, rank, taps = 40, 24, 5, 4
    lengths, slots = [3, 1, 9], [2, 0, 3]
    q_start_loc, seq_of_token = _meta(lengths)
    slot_t = torch.tensor(slots, dtype=torch.int32, device="cuda")
    tokens = sum(lengths)
    h = torch.randn(tokens, width, generator=g)
    before = torch.randn(5, width, generator=g)
    mu = torch.rand(5, width, generator=g)
    state = before.clone().cuda()
    mixes = ops.shift_mix(h.cuda(), state, mu.cuda(), seq_of_token, slot_t, q_start_loc)
    prev = h.clone()
    prev[1:] = h[:-1]
    first = 0
    for length, slot in zip(lengths, slots):
        prev[first] = before[slot]
        first += length
    want = h[None] + (prev - h)[None] * mu[:, None, :]
    assert torch.allclose(mixes.cpu(), want, atol=1e-6)
    low = torch.randn(tokens, rank, generator=g)
    w2, w0 = torch.randn(channels, rank, generator=g), torch.randn(channels, generator=g)
    decay = ops.time_decay(low.cuda(), w2.t().contiguous().cuda(), w0.cuda(), h.cuda(), state, seq_of_token, slot_t, q_start_loc)
    assert torch.allclose(decay.cpu(), torch.exp(-torch.exp(torch.tanh(low) @ w2.t() + w0)), atol=1e-6, rtol=1e-5)
    kept = before.clone()
    first = 0
    for length, slot in zip(lengths, slots):
        kept[slot] = h[first + length - 1]
        first += length
    assert torch.equal(state.cpu(), kept)
    # the convolution: silu behind the taps, float32 out of either type, and the state moved on behind it
    x = torch.randn(tokens, channels + 8, generator=g)
    taps_w, bias = torch.randn(channels, taps, generator=g), torch.randn(channels, generator=g)
    past = torch.randn(5, taps - 1, channels, generator=g)
    past_gpu = past.clone().cuda()
    view = x.cuda()[:, 4: 4 + channels]
    out = ops.causal_conv(view, taps_w.cuda(), bias.cuda(), past_gpu, seq_of_token, slot_t, q_start_loc, activation="silu",
                          out_dtype=torch.float32)
    ops.conv_keep(view, past_gpu, slot_t, q_start_loc, len(lengths), taps)
    first = 0
    for length, slot in zip(lengths, slots):
        rows = torch.cat([past[slot], x[first: first + length, 4: 4 + channels]], dim=0)
        for t in range(length):
            want_t = torch.nn.functional.silu((rows[t: t + taps] * taps_w.t()).sum(0) + bias)
            assert torch.allclose(out[first + t].cpu(), want_t, atol=1e-5), (slot, t)
        assert torch.equal(past_gpu[slot].cpu(), rows[-(taps - 1):])
        first += length
