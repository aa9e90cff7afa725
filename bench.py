#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens per second of a Qwen2.5 shape
(default: the 3B one) with random weights, plus prefill and roofline figures.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096]
                    [--shape 0.5b|3b|7b|14b|32b|72b] [--layers N] [--long-contexts 32768]
                    [--mixed-portions 16,64,248] [--other-shapes 7b,14b]
    python bench.py --design polosun|givizen|nokipel|senuvik [--design-shapes 3b,7b] [--design-layers 12]

A "step" is one decode step of the whole engine (scheduler iteration: plan,
step function, sampling, token hand-over).  Protocol after the reference's
benchmark (benchmarks/run.py:3-8, 205-207, 241-256): a fresh engine per
measured point, two unmeasured warm-up runs, three measured runs, every run
reported and the median taken; wall-clock output tokens per second; prompts are
seeded uniform-random token ids, EOS is ignored.

A *run* of the headline figure is a window of exactly K decode steps between two
``torch.cuda.synchronize()``; the windows follow one another in the same batch
of requests, after W untimed steps, and the last one ends at ``--context``
tokens, so all of them sit at the heavy end of the range that the configuration
states ("2,048-token prefill, then decode to 4,096").  The whole range is
measured beside it (``range``): prompts of ``--prefill-tokens``, then every
decode step up to ``--context``, one warm-up run and three measured ones.
``prefill`` is one prompt of ``--prefill-tokens`` run to its first token.
``mixed`` is the time of the steps that chunked serving meets: the batch's decode
tokens beside one portion of a further prompt (``--mixed-portions``).  ``points``
holds decode at batch 1 and 64, at the main batch behind ``--long-contexts``
tokens, and, for the ``--other-shapes`` of the family, decode at the main batch
and context and the prefill, each with its share of the roofline in
``points_frac`` (the bytes and flops of its own shape).  ONE JSON line is printed.

``--design polosun`` measures something else and leaves the above as it is: the
Polosun design (layers of retention, latent attention and gated linear
recurrence in turn, each with a dense feed-forward) beside the Qwen2.5 decoder
of equal width, feed-forward size, vocabulary and layer count, both with
``--design-layers`` layers and random weights: prefill of ``--prefill-tokens``
tokens and decode at batch 1, ``--batch`` and 64 behind ``--context`` tokens,
each with its share of the roofline of its own bytes and flops.  It prints one
JSON line of its own.  ``--design givizen`` does the same for the Givizen design
(window attention with shaped scores of two kinds in turn, each layer with
routed experts and a shared one whose active sizes add up to the Qwen2.5
shape's feed-forward).  ``--design nokipel`` measures the Nokipel design (three
layers of lightning attention to one of chunked softmax attention, dense
bounded feed-forwards and routed experts in turn) beside the Givizen model of
equal width, head sizes, expert sizes, vocabulary and layer count, the closest
of the engine's models: the same attention and expert kernels with other
options.  ``--design senuvik`` measures the Senuvik design (window attention
with kept first tokens, a state-space mixer, causal attention beside time
mixing, and window attention on another layer's keys in turn; a dense
feed-forward and routed experts) beside the Nokipel model of equal width, head
sizes, expert sizes, vocabulary and layer count, the closest of the engine's
models: memories of fixed size beside attention, dense and routed
feed-forwards.
"""

from __future__ import annotations

import argparse
import gc
import json
import statistics
import sys
import time

# MI355X published peaks.
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

SLACK = 16  # tokens a request may run past the nominal context (requests start decoding a step or two apart)
WARM_WINDOWS = 2
MEASURED_WINDOWS = 3
PAGE = 16


def linear_params_per_layer(c) -> int:
    q = c.num_attention_heads * c.head_dim
    kv = c.num_key_value_heads * c.head_dim
    return c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size


def decode_bytes(c, layers: int, batch: int, context: float, elem: int) -> float:
    """Bytes one decode step has to read: every weight once, and the cache of the live requests."""
    weights = layers * (linear_params_per_layer(c) + 2 * c.hidden_size
                        + (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim) * elem
    weights += c.vocab_size * c.hidden_size * elem + c.hidden_size * elem  # the head (tied or not: read once) + final norm
    kv = batch * context * layers * 2 * c.num_key_value_heads * c.head_dim * elem
    return weights + kv


def prefill_flops(c, layers: int, tokens: int) -> float:
    linears = 2.0 * tokens * layers * linear_params_per_layer(c)
    attention = layers * 2 * 2 * (tokens * (tokens + 1) / 2) * c.head_dim * c.num_attention_heads
    head = 2.0 * c.hidden_size * c.vocab_size
    return linears + attention + head


def make_engine(config, dtype, batch, context, prefill_tokens, seed=0):
    from cie_amd import Engine

    per_request = -(-(context + SLACK) // PAGE) * PAGE
    kv_tokens = max(batch * per_request, -(-prefill_tokens // PAGE) * PAGE) + 4 * PAGE
    return Engine(
        config=config, seed=seed, dtype=dtype, page_size=PAGE, kv_tokens=kv_tokens,
        max_running=max(batch, 1), max_queue_size=max(batch, 1) + 1, max_model_len=context + SLACK,
        max_output_tokens=context, token_budget=max(2048, batch), prefill_chunk=2048,
        prefix_cache_pages=0, draw_device="cuda",
        # fill all caches before decoding starts, so that the timed steps are pure decode steps
        plan_order=lambda standing: (standing.decoding,),
    )


def random_prompts(config, count: int, length: int, seed: int) -> list[list[int]]:
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, config.vocab_size, (length,), generator=g).tolist() for _ in range(count)]


def decode_windows(engine, config, batch: int, context: int, steps: int, warmup: int, seed: int):
    """``batch`` requests whose last window ends at ``context``: W untimed steps, then
    ``WARM_WINDOWS`` unmeasured and ``MEASURED_WINDOWS`` measured windows of exactly ``steps`` steps.
    Returns [(seconds, mean context of the window)] of the measured ones."""
    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    windows = WARM_WINDOWS + MEASURED_WINDOWS
    prompt_len = context - warmup - windows * steps
    if prompt_len < 1:
        raise ValueError(f"context {context} too short for {warmup} + {windows} x {steps} steps")
    gen = GenerationConfig(max_output_tokens=warmup + windows * steps + SLACK, eos_token_id=None)
    requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, prompt_len, seed)]
    while any(r.state is not RequestState.DECODING for r in requests):
        engine.step()  # prefill portions; the last one yields each request's first token
    for _ in range(warmup - 1):
        engine.step()
    measured = []
    for window in range(windows):
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        if window >= WARM_WINDOWS:
            measured.append((elapsed, sum(r.cached for r in requests) / batch - steps / 2.0))
    for r in requests:
        # (with decode steps started ahead of their tokens, the last step's token is still on its way)
        assert not r.is_final and len(r.output) >= warmup + windows * steps - 1, (r.state, len(r.output))
        engine.scheduler.cancel(r)
    return measured


def decode_range(engine, config, batch: int, first: int, last: int, seed: int, warm_steps: int = 48):
    """Prompts of ``first`` tokens, then every decode step until the requests hold ``last`` tokens:
    one short unmeasured run, ``MEASURED_WINDOWS`` measured ones.  Returns [(seconds, decode steps)]."""
    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    out = []
    for run in range(1 + MEASURED_WINDOWS):
        tokens = min(warm_steps, last - first) if run == 0 else last - first
        gen = GenerationConfig(max_output_tokens=tokens, eos_token_id=None)
        requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, first, seed + run)]
        while any(r.state is not RequestState.DECODING for r in requests):
            engine.step()
        torch.cuda.synchronize()
        start = time.perf_counter()
        while engine.has_work():
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert all(len(r.output) == tokens for r in requests)
        if run:
            out.append((elapsed, tokens - 1))  # the first token came with the prompt
    return out


def mixed_steps(engine, config, batch: int, context: int, portions: list[int], seed: int, steps: int = 24):
    """``batch`` requests decoding near ``context`` tokens; for each portion size, steps that carry
    their tokens and one portion of a long prompt.  Returns {portion: median seconds per step}."""
    import dataclasses

    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    settle = 4
    decoded = (len(portions) + 1) * (steps + 2 * settle + 4) + SLACK
    gen = GenerationConfig(max_output_tokens=decoded, eos_token_id=None)
    requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, context - decoded, seed)]
    while any(r.state is not RequestState.DECODING for r in requests):
        engine.step()
    base = engine.scheduler.config
    out = {}
    for portion in portions:
        # the scheduler cuts the long prompt into portions of this size beside the decode tokens
        engine.scheduler.config = dataclasses.replace(base, token_budget=batch + portion, prefill_chunk=portion)
        prompt = random_prompts(config, 1, portion * (steps + settle + 2), seed + portion)[0]
        long = engine.submit(prompt, GenerationConfig(max_output_tokens=1, eos_token_id=None))
        for _ in range(settle):  # (a shape is captured the second time it comes)
            engine.step()
        seconds = []
        for _ in range(steps):
            torch.cuda.synchronize()
            start = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            seconds.append(time.perf_counter() - start)
        assert not long.is_final and all(r.state is RequestState.DECODING for r in requests)
        out[portion] = statistics.median(seconds)
        while not long.is_final:
            engine.step()
    engine.scheduler.config = base
    for r in requests:
        assert not r.is_final
        engine.scheduler.cancel(r)
    return out


def time_prefill(engine, config, tokens: int, seed: int) -> list[float]:
    """Seconds of each measured run: one prompt from submission to its first token."""
    import torch

    from cie_amd import GenerationConfig

    seconds = []
    prompts = random_prompts(config, WARM_WINDOWS + MEASURED_WINDOWS, tokens, seed)
    for run, prompt in enumerate(prompts):
        request = engine.submit(prompt, GenerationConfig(max_output_tokens=1, eos_token_id=None))
        torch.cuda.synchronize()
        start = time.perf_counter()
        while not request.is_final:
            engine.step()
        torch.cuda.synchronize()
        if run >= WARM_WINDOWS:
            seconds.append(time.perf_counter() - start)
    return seconds


def polosun_raw(shape: dict, layers: int) -> dict:
    """A Polosun configuration with the width, feed-forward size and vocabulary of a Qwen2.5 shape and layers of
    realistic proportions: retention heads of 128 x 256, latent attention with heads of 128 + 32 whose cache entry
    (a latent of 96 and a turned part of 32) fills one 128-wide head of the attention kernels, a gated recurrence as
    wide as the model in blocks of 256 channels with four taps."""
    width = shape["hidden_size"]
    mlp = {"kind": "dense", "ff": shape["intermediate_size"]}
    kinds = [
        {"type": "retention", "mlp": mlp,
         "mixer": {"heads": width // 256, "dim": 128, "vdim": 256, "rot": {"base": 10000.0, "dims": 128},
                   "decay": [1.0 - 2.0 ** (-5 - 3 * h / max(width // 256 - 1, 1)) for h in range(width // 256)]}},
        {"type": "latent_attention", "mlp": mlp,
         "mixer": {"heads": width // 128, "dim": 128, "rot_dim": 32, "vdim": 128, "kv_rank": 96, "scale": 160 ** -0.5,
                   "rot": {"base": 1000000.0, "dims": 32,
                           "scaling": {"factor": 4.0, "fast": 32.0, "original": 8192, "slow": 1.0}}}},
        {"type": "rglru", "mlp": mlp, "mixer": {"width": width, "blocks": width // 256, "conv": 4}},
    ]
    return {"architecture": "Polosun", "vocab": shape["vocab_size"], "width": width, "residual_mult": 0.5,
            "norm": {"eps": 1e-6}, "layers": [kinds[i % 3] for i in range(layers)]}


def polosun_costs(config, batch: int, context: float, tokens: int, elem: int) -> tuple[float, float]:
    """(bytes one decode step has to move, flops of a prefill of ``tokens`` tokens) for a Polosun configuration:
    every weight once (the embedding is only looked up), each request's latent cache read in both of its layouts,
    each retention memory and recurrence state read and written in float32; products at two flops per weight and
    token, attention over the latent entries, the memories' updates and read-outs."""
    from cie_amd.parts.model import expected_tensors

    expected = expected_tensors(config.model_spec())
    weights = sum(int(__import__("math").prod(spec.shape)) for name, spec in expected.items() if name != "embed")
    head = config.vocab_size * config.hidden_size
    moved, attention = float(weights * elem), 0.0
    for layer in config.raw["layers"]:
        m = layer["mixer"]
        if layer["type"] == "latent_attention":
            entry = next(size for size in (32, 64, 96, 128, 256) if size >= m["kv_rank"] + m["rot_dim"])
            moved += batch * context * 2 * entry * elem
            attention += 2 * 2 * (tokens * (tokens + 1) / 2) * entry * m["heads"]
        elif layer["type"] == "retention":
            moved += batch * 2 * m["heads"] * m["dim"] * m["vdim"] * 4
            attention += 2 * 2 * tokens * m["heads"] * m["dim"] * m["vdim"]
        else:
            moved += batch * 2 * m["width"] * m["conv"] * 4
    return moved, 2.0 * tokens * (weights - head) + 2.0 * head + attention


GIVIZEN_EXPERTS, GIVIZEN_TOP = 32, 4
GIVIZEN_WINDOWS = (1024, 4096)


def givizen_raw(shape: dict, layers: int) -> dict:
    """A Givizen configuration with the width, vocabulary, head counts and head size of a Qwen2.5 shape: layers of
    the two attention kinds in turn (windows of 1,024 and 4,096 tokens), each with 32 experts of which a token uses
    4, and a shared expert; the four experts and the shared one together are as large as the shape's feed-forward."""
    width = shape["hidden_size"]
    heads, kv_heads = shape["num_attention_heads"], shape["num_key_value_heads"]
    dim = width // heads
    expert_ff = shape["intermediate_size"] // (2 * GIVIZEN_TOP) // 64 * 64
    shared_ff = shape["intermediate_size"] - GIVIZEN_TOP * expert_ff
    mlp = {"kind": "moe", "router": {"experts": GIVIZEN_EXPERTS, "top": GIVIZEN_TOP},
           "expert": {"ff": expert_ff, "limit": 7.0}, "shared": {"ff": shared_ff, "limit": 7.0}}
    common = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
              "q_temp": {"coef": 0.1, "every": 1024}}
    kinds = [
        {"type": "attention", "mlp": mlp, "mixer": {**common, "mask": {"size": GIVIZEN_WINDOWS[0]}}},
        {"type": "attention_2", "mlp": mlp, "mixer": {**common, "mask": {"size": GIVIZEN_WINDOWS[1]}, "softcap": 50.0}},
    ]
    return {"architecture": "Givizen", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "logit_softcap": 30.0, "layers": [kinds[i % 2] for i in range(layers)]}


def givizen_costs(config, batch: int, context: float, tokens: int, elem: int) -> tuple[float, float]:
    """(bytes one decode step has to move, flops of a prefill of ``tokens`` tokens) for a Givizen configuration:
    every weight that a step touches once (of a layer's experts, the ones that ``batch`` tokens choosing ``top`` of
    them at random are expected to hit), each request's keys and values inside the layer's window; products at two
    flops per active weight and token, attention over the keys each token sees."""
    width, vocab = config.hidden_size, config.vocab_size
    moved = float(vocab * width * elem)
    flops = 2.0 * vocab * width
    for layer in config.raw["layers"]:
        m, mlp = layer["mixer"], layer["mlp"]
        mixer = width * (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"]) + m["heads"] * m["vdim"])
        if layer["type"] == "attention_2":
            mixer += width * m["heads"]
        experts, top = mlp["router"]["experts"], mlp["router"]["top"]
        one = 3 * width * mlp["expert"]["ff"]
        shared = 3 * width * mlp["shared"]["ff"] if mlp.get("shared") else 0
        hit = experts * (1.0 - (1.0 - top / experts) ** batch)
        moved += (mixer + width * experts + shared + hit * one) * elem
        seen = min(context, m["mask"]["size"])
        moved += batch * seen * m["kv_heads"] * (m["dim"] + m["vdim"]) * elem
        flops += 2.0 * tokens * (mixer + width * experts + shared + top * one)
        window = min(tokens, m["mask"]["size"])
        pairs = window * (window + 1) / 2 + (tokens - window) * window
        flops += 2.0 * pairs * m["heads"] * (m["dim"] + m["vdim"])
    return moved, flops


NOKIPEL_IDENTITY = 2
NOKIPEL_GROUPS = (4, 2)


def nokipel_raw(shape: dict, layers: int) -> dict:
    """A Nokipel configuration with the width, vocabulary, head counts and head size of a Qwen2.5 shape: of every
    four layers three have lightning attention (heads of 128 x 128, decays spread from 1 - 2^-5 to 1 - 2^-8) and one
    has softmax attention in chunks of as many tokens as Givizen's shorter window, with a rotation over half of each
    head; dense feed-forwards of the shape's size and routed ones take turns: 30 experts and 2 identity experts in 4
    groups of which 2 are kept, 4 per token, experts and the shared one of Givizen's sizes; norms in 2 groups."""
    width = shape["hidden_size"]
    heads, kv_heads = shape["num_attention_heads"], shape["num_key_value_heads"]
    dim = width // heads
    expert_ff = shape["intermediate_size"] // (2 * GIVIZEN_TOP) // 64 * 64
    shared_ff = shape["intermediate_size"] - GIVIZEN_TOP * expert_ff
    dense = {"kind": "dense", "ff": shape["intermediate_size"], "limit": 7.0}
    routed = {"kind": "moe", "expert": {"ff": expert_ff}, "shared": {"ff": shared_ff},
              "router": {"experts": GIVIZEN_EXPERTS - NOKIPEL_IDENTITY, "identity": NOKIPEL_IDENTITY, "top": GIVIZEN_TOP,
                         "scale": 2.0, "groups": {"count": NOKIPEL_GROUPS[0], "keep": NOKIPEL_GROUPS[1]}}}
    memories = width // 128
    lightning = {"heads": memories, "dim": 128, "vdim": 128,
                 "decay": [1.0 - 2.0 ** (-5 - 3 * h / max(memories - 1, 1)) for h in range(memories)]}
    attention = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                 "mask": {"size": GIVIZEN_WINDOWS[0]}, "rot": {"base": 1000000.0, "dims": dim // 2}}
    kinds = [
        {"type": "lightning", "mixer": lightning, "mlp": dense},
        {"type": "lightning", "mixer": lightning, "mlp": routed},
        {"type": "lightning", "mixer": lightning, "mlp": dense},
        {"type": "attention", "mixer": attention, "mlp": routed},
    ]
    return {"architecture": "Nokipel", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6, "groups": 2},
            "embedding": {"scale": 1.0}, "layers": [kinds[i % 4] for i in range(layers)]}


def nokipel_costs(config, batch: int, context: float, tokens: int, elem: int) -> tuple[float, float]:
    """(bytes one decode step has to move, flops of a prefill of ``tokens`` tokens) for a Nokipel configuration
    without a loop: every weight that a step touches once (of a layer's experts, the ones that ``batch`` tokens
    choosing ``top`` of all router outputs at random are expected to hit; identity experts have none), each
    request's keys and values inside the token's chunk, each lightning memory read and written in float32; products
    at two flops per active weight and token, attention over the keys each token sees, the memories' updates and
    read-outs."""
    width, vocab = config.hidden_size, config.vocab_size
    moved = float(vocab * width * elem)
    flops = 2.0 * vocab * width
    for layer in config.raw["layers"]:
        m, mlp = layer["mixer"], layer["mlp"]
        if layer["type"] == "lightning":
            mixer = width * m["heads"] * (2 * m["dim"] + 3 * m["vdim"])
            moved += batch * 2 * m["heads"] * m["dim"] * m["vdim"] * 4
            flops += 2.0 * 2 * tokens * m["heads"] * m["dim"] * m["vdim"]
        else:
            mixer = width * (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"]) + m["heads"] * m["vdim"])
            size = m["mask"]["size"] if m.get("mask") else None
            seen = context if size is None else context % size + 1
            moved += batch * seen * m["kv_heads"] * (m["dim"] + m["vdim"]) * elem
            whole, rest = (tokens // size, tokens % size) if size else (0, tokens)
            pairs = whole * size * (size + 1) / 2 + rest * (rest + 1) / 2
            flops += 2.0 * pairs * m["heads"] * (m["dim"] + m["vdim"])
        if mlp is None:
            active = touched = 0.0
        elif mlp["kind"] == "dense":
            active = touched = 3.0 * width * mlp["ff"]
        else:
            router = mlp["router"]
            experts, top = router["experts"], router["top"]
            outputs = experts + router.get("identity", 0)
            one = 3 * width * mlp["expert"]["ff"]
            shared = 3 * width * mlp["shared"]["ff"] + width if mlp.get("shared") else 0
            hit = experts * (1.0 - (1.0 - top / outputs) ** batch)
            touched = width * outputs + shared + hit * one
            active = width * outputs + shared + top * experts / outputs * one
        moved += (mixer + touched) * elem
        flops += 2.0 * tokens * (mixer + active)
    return moved, flops


SENUVIK_WINDOW, SENUVIK_KEPT = 1024, 64


def senuvik_raw(shape: dict, layers: int) -> dict:
    """A Senuvik configuration with the width, vocabulary, head counts and head size of a Qwen2.5 shape.  Of every
    four layers the first has window attention (1,024 tokens beside 64 kept first ones, a rotation over half of each
    head) and a dense feed-forward of the shape's size, the second a state-space mixer twice as wide as the stream
    (heads of 64 numbers, memories of 128 rows, 8 groups), the third causal attention beside time mixing (heads of
    64), and the fourth window attention on the first layer's keys and values; these three have routed feed-forwards
    of Givizen's sizes (32 experts, 4 per token, a gated shared expert)."""
    width = shape["hidden_size"]
    heads, kv_heads = shape["num_attention_heads"], shape["num_key_value_heads"]
    dim = width // heads
    expert_ff = shape["intermediate_size"] // (2 * GIVIZEN_TOP) // 64 * 64
    shared_ff = shape["intermediate_size"] - GIVIZEN_TOP * expert_ff
    dense = {"kind": "dense", "ff": shape["intermediate_size"]}
    routed = {"kind": "moe", "expert": {"ff": expert_ff}, "shared": {"ff": shared_ff},
              "router": {"experts": GIVIZEN_EXPERTS, "top": GIVIZEN_TOP}}
    window = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
              "mask": {"size": SENUVIK_WINDOW, "keep_first": SENUVIK_KEPT},
              "rot": {"base": 1000000.0, "dims": dim // 2, "scaling": {"factor": 4.0}}}
    space = {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 8, "conv": 4, "norm_groups": 8}
    pair = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "softcap": 50.0,
                     "rot": {"base": 1000000.0, "dims": dim,
                             "scaling": {"factor": 4.0, "original": 8192, "fast": 32.0, "slow": 1.0}}},
            "right": {"heads": width // 64, "dim": 64}, "left_scale": 0.5, "right_scale": 0.5}
    out = []
    for i in range(layers):
        kind = i % 4
        if kind == 0:
            out.append({"type": "attention", "mixer": dict(window), "mlp": dense})
        elif kind == 1:
            out.append({"type": "mamba2", "mixer": space, "mlp": routed})
        elif kind == 2:
            out.append({"type": "parallel", "mixer": pair, "mlp": routed})
        else:
            out.append({"type": "attention", "mixer": dict(window, kv_from=i - 3), "mlp": routed})
    return {"architecture": "Senuvik", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6}, "layers": out}


SENUVIK_DECAY_RANK = 64   # (the rank of the decay's two small products is the checkpoint's; random weights draw this)


def senuvik_costs(config, batch: int, context: float, tokens: int, elem: int) -> tuple[float, float]:
    """(bytes one decode step has to move, flops of a prefill of ``tokens`` tokens) for a Senuvik configuration:
    every weight that a step touches once (of a layer's experts, the ones that ``batch`` tokens choosing ``top`` of
    them at random are expected to hit), each request's keys and values inside the window and among the kept first
    tokens (once for the layer that writes them and once for every layer that reads them), every memory read and
    written in float32; products at two flops per active weight and token, attention over the keys a token sees,
    the memories' updates and read-outs."""
    width, vocab = config.hidden_size, config.vocab_size
    moved = float(vocab * width * elem)
    flops = 2.0 * vocab * width

    def attention(m, size, keep):
        nonlocal moved, flops
        seen = context if size is None else min(context, size + keep)
        moved += batch * seen * m["kv_heads"] * (m["dim"] + m["vdim"]) * elem
        if size is None:
            pairs = tokens * (tokens + 1) / 2
        else:
            reach = min(tokens, size)
            pairs = reach * (reach + 1) / 2 + (tokens - reach) * (reach + keep)
        flops += 2.0 * pairs * m["heads"] * (m["dim"] + m["vdim"])

    for layer in config.raw["layers"]:
        m, mlp = layer["mixer"], layer["mlp"]
        if layer["type"] == "attention":
            own = m.get("kv_from") is None
            mixer = width * (m["heads"] * m["dim"] + m["heads"] * m["vdim"])
            mixer += width * m["kv_heads"] * (m["dim"] + m["vdim"]) if own else 0
            attention(m, m["mask"]["size"], m["mask"].get("keep_first", 0))
        elif layer["type"] == "mamba2":
            inner = m["heads"] * m["vdim"]
            mixer = width * (2 * inner + 2 * m["groups"] * m["state"] + m["heads"]) + inner * width
            moved += batch * 2 * m["heads"] * m["state"] * m["vdim"] * 4
            flops += 2.0 * 2 * tokens * m["heads"] * m["state"] * m["vdim"]
        else:
            left, right = m["left"], m["right"]
            mixer = width * (left["heads"] * left["dim"] + left["kv_heads"] * (left["dim"] + left["vdim"])
                             + left["heads"] * left["vdim"] + left["heads"])
            channels = right["heads"] * right["dim"]
            mixer += 5 * width * channels + SENUVIK_DECAY_RANK * (width + channels)
            attention(left, None, 0)
            moved += batch * 2 * right["heads"] * right["dim"] * right["dim"] * 4
            flops += 2.0 * 2 * tokens * right["heads"] * right["dim"] * right["dim"]
        if mlp is None:
            active = touched = 0.0
        elif mlp["kind"] == "dense":
            active = touched = 3.0 * width * mlp["ff"]
        else:
            experts, top = mlp["router"]["experts"], mlp["router"]["top"]
            one = 3 * width * mlp["expert"]["ff"]
            shared = 3 * width * mlp["shared"]["ff"] + width if mlp.get("shared") else 0
            hit = experts * (1.0 - (1.0 - top / experts) ** batch)
            touched = width * experts + shared + hit * one
            active = width * experts + shared + top * one
        moved += (mixer + touched) * elem
        flops += 2.0 * tokens * (mixer + active)
    return moved, flops


def compare_designs(args) -> int:
    """``--design polosun``, ``--design givizen``, ``--design nokipel`` or ``--design senuvik``: see the module's text."""
    import torch

    from cie_amd.config import GivizenConfig, NokipelConfig, PolosunConfig, Qwen2Config, SenuvikConfig
    from cie_amd.workloads import SHAPES

    elem = 2 if args.dtype == "bf16" else 4
    steps, warmup, layers = args.steps, max(args.warmup, 1), args.design_layers
    out = {}
    for name in [n for n in args.design_shapes.split(",") if n]:
        shape = SHAPES[name]
        if args.design == "nokipel":
            designs = {"nokipel": NokipelConfig.from_hf_config(nokipel_raw(shape, layers)),
                       "givizen": GivizenConfig.from_hf_config(givizen_raw(shape, layers))}
        elif args.design == "senuvik":
            designs = {"senuvik": SenuvikConfig.from_hf_config(senuvik_raw(shape, layers)),
                       "nokipel": NokipelConfig.from_hf_config(nokipel_raw(shape, layers))}
        else:
            designs = {
                args.design: (PolosunConfig.from_hf_config(polosun_raw(shape, layers)) if args.design == "polosun"
                              else GivizenConfig.from_hf_config(givizen_raw(shape, layers))),
                "qwen2": Qwen2Config.from_hf_config(dict(shape, num_hidden_layers=layers)),
            }
        out[name] = {}
        for design, config in designs.items():
            def costs(batch, context):
                if design == "polosun":
                    return polosun_costs(config, batch, context, args.prefill_tokens, elem)
                if design == "givizen":
                    return givizen_costs(config, batch, context, args.prefill_tokens, elem)
                if design == "nokipel":
                    return nokipel_costs(config, batch, context, args.prefill_tokens, elem)
                if design == "senuvik":
                    return senuvik_costs(config, batch, context, args.prefill_tokens, elem)
                return (decode_bytes(config, layers, batch, context, elem), prefill_flops(config, layers, args.prefill_tokens))

            record = {}
            print(f"[bench] {design} at the {name} widths, {layers} layers: prefill of {args.prefill_tokens}", file=sys.stderr, flush=True)
            engine = make_engine(config, args.dtype, 1, args.prefill_tokens + 1, args.prefill_tokens)
            seconds = statistics.median(time_prefill(engine, config, args.prefill_tokens, seed=99))
            del engine
            gc.collect()
            torch.cuda.empty_cache()
            record["prefill"] = {"tokens_per_s": round(args.prefill_tokens / seconds, 1), "ms": round(seconds * 1e3, 3),
                                 "frac": round(costs(1, 1)[1] / seconds / PEAK_FLOPS[args.dtype], 4)}
            for batch in sorted({1, args.batch, 64}):
                print(f"[bench] {design} at the {name} widths: decode, batch {batch}, context {args.context}", file=sys.stderr, flush=True)
                engine = make_engine(config, args.dtype, batch, args.context, args.prefill_tokens)
                measured = decode_windows(engine, config, batch, args.context, steps, warmup, seed=batch)
                del engine
                gc.collect()
                torch.cuda.empty_cache()
                taken, mean_context = sorted(measured)[len(measured) // 2]
                record[f"decode_b{batch}"] = {
                    "tokens_per_s": round(batch * steps / taken, 2), "ms_per_step": round(taken / steps * 1e3, 4),
                    "frac": round(costs(batch, mean_context)[0] / (taken / steps) / 1e9 / HBM_GBPS, 4)}
            out[name][design] = record
    givizen_layers = (f"attention (window {GIVIZEN_WINDOWS[0]}) and attention_2 (window {GIVIZEN_WINDOWS[1]}) in turn, each "
                      f"with {GIVIZEN_EXPERTS} experts, {GIVIZEN_TOP} per token, and a shared expert")
    nokipel_layers = (f"lightning + dense, lightning + experts, lightning + dense, attention (chunks of "
                      f"{GIVIZEN_WINDOWS[0]}) + experts in turn; {GIVIZEN_EXPERTS - NOKIPEL_IDENTITY} experts and "
                      f"{NOKIPEL_IDENTITY} identity experts in {NOKIPEL_GROUPS[0]} groups ({NOKIPEL_GROUPS[1]} kept), "
                      f"{GIVIZEN_TOP} per token, and a gated shared expert")
    senuvik_layers = (f"window attention ({SENUVIK_WINDOW} tokens beside {SENUVIK_KEPT} kept first ones) + dense, state space + "
                      f"experts, causal attention beside time mixing + experts, window attention on the first layer's keys "
                      f"+ experts in turn; {GIVIZEN_EXPERTS} experts, {GIVIZEN_TOP} per token, and a gated shared expert")
    beside = ("the Givizen model of equal width, head and expert sizes" if args.design == "nokipel"
              else "the Nokipel model of equal width, head and expert sizes" if args.design == "senuvik"
              else "the Qwen2.5 decoder of equal width, feed-forward")
    print(json.dumps({
        "metric": f"{args.design.capitalize()} beside {beside}, vocabulary and {layers} layers",
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "dtype": args.dtype,
        "data": "synthetic (seeded uniform-random token ids, random weights N(0, 0.02))",
        "config": {"layers": layers, "context": args.context, "prefill_tokens": args.prefill_tokens, "page_size": PAGE,
                   "design_layers": ("retention, latent_attention, rglru in turn, each with a dense feed-forward"
                                     if args.design == "polosun" else givizen_layers if args.design == "givizen" else
                                     senuvik_layers + "; beside it Nokipel: " + nokipel_layers if args.design == "senuvik" else
                                     nokipel_layers + "; beside it Givizen: " + givizen_layers)},
        "shapes": out,
    }))
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--shape", default="3b", choices=["0.5b", "3b", "7b", "14b", "32b", "72b"])
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--no-range", action="store_true", help="skip the run over the whole range of contexts")
    parser.add_argument("--long-contexts", default=None,
                        help="further decode points of the main batch, e.g. 16384,32768 (default: 32768; none with --no-points)")
    parser.add_argument("--mixed-portions", default=None,
                        help="also time steps of the batch's decode tokens beside a prompt portion of these sizes "
                             "(default 16,64,248; '' for none, as with --no-points)")
    parser.add_argument("--other-shapes", default="7b,14b",
                        help="further shapes whose decode at the main batch and context and whose prefill go into the points ('' for none)")
    parser.add_argument("--design", default=None, choices=["polosun", "givizen", "nokipel", "senuvik"],
                        help="instead of the default record: this design beside the Qwen2.5 decoder of equal size "
                             "(nokipel: beside the Givizen model of equal size; senuvik: beside the Nokipel model)")
    parser.add_argument("--design-shapes", default="3b,7b", help="the Qwen2.5 shapes whose sizes the comparison takes")
    parser.add_argument("--design-layers", type=int, default=12, help="layers of both models in the comparison")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not run (this engine is single-GPU)")
        return 2

    if args.design is not None:
        return compare_designs(args)

    import torch

    from cie_amd.config import Qwen2Config
    from cie_amd.workloads import SHAPES

    shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    layers = args.layers or full_layers
    config = Qwen2Config.from_hf_config(dict(shape, num_hidden_layers=layers))
    elem = 2 if args.dtype == "bf16" else 4
    steps, warmup = args.steps, max(args.warmup, 1)

    def release() -> None:
        # (an engine's memory has to be back before the next engine is built: the large shapes fit once)
        gc.collect()
        torch.cuda.empty_cache()

    def say(text: str) -> None:
        print(f"[bench] {text}", file=sys.stderr, flush=True)

    def point(batch: int, context: int, config=config, layers=layers, label: str = ""):
        """(tokens/s of each measured window, the median window's ms per step and roofline share)."""
        context = min(context, config.max_position_embeddings - SLACK)  # (the last positions are the slack's)
        say(f"decode{label}, batch {batch}, context {context}")
        engine = make_engine(config, args.dtype, batch, context, args.prefill_tokens)
        measured = decode_windows(engine, config, batch, context, steps, warmup, seed=batch)
        del engine
        release()
        rates = [batch * steps / seconds for seconds, _ in measured]
        seconds, mean_context = sorted(measured)[len(measured) // 2]
        achieved = decode_bytes(config, layers, batch, mean_context, elem) / (seconds / steps) / 1e9
        return rates, seconds / steps * 1e3, achieved

    def prefill_point(config=config, layers=layers, label: str = ""):
        """(seconds of each measured run, the step's flops) of one prompt run to its first token."""
        say(f"prefill{label} of {args.prefill_tokens} tokens")
        engine = make_engine(config, args.dtype, 1, args.prefill_tokens + 1, args.prefill_tokens)
        seconds = time_prefill(engine, config, args.prefill_tokens, seed=99)
        del engine
        release()
        return seconds, prefill_flops(config, layers, args.prefill_tokens)

    rates, ms_per_step, achieved = point(args.batch, args.context)
    name = f"Qwen2.5-{args.shape.upper()} shape"
    line = {
        "metric": f"decode tokens/s, {name}, batch {args.batch}, context to {args.context}",
        "value": round(statistics.median(rates), 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic (seeded uniform-random token ids, random weights N(0, 0.02))",
        "config": {
            "model": f"{name} (Qwen2ForCausalLM)", "layers": layers, "layers_full": full_layers,
            "hidden": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate": config.intermediate_size, "vocab": config.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": args.prefill_tokens,
            "page_size": PAGE, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings, "attention_bias": config.attention_bias,
            "parallelism": "single GPU",
        },
        "protocol": f"fresh engine per point, {WARM_WINDOWS} unmeasured and {MEASURED_WINDOWS} measured windows of "
                    f"{steps} steps after {warmup} warm-up steps; value is the median window",
        "runs": [round(r, 2) for r in rates],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    if not args.no_range and args.context > args.prefill_tokens + 1:
        say(f"decode over the range {args.prefill_tokens} to {args.context}")
        engine = make_engine(config, args.dtype, args.batch, args.context, args.prefill_tokens)
        runs = decode_range(engine, config, args.batch, args.prefill_tokens, args.context, seed=7)
        del engine
        release()
        range_rates = [args.batch * n / seconds for seconds, n in runs]
        seconds, n = sorted(runs)[len(runs) // 2]
        mean_context = (args.prefill_tokens + args.context) / 2.0
        through = decode_bytes(config, layers, args.batch, mean_context, elem) / (seconds / n) / 1e9
        line["range"] = {
            "from": args.prefill_tokens, "to": args.context, "steps": n,
            "value": round(statistics.median(range_rates), 2), "runs": [round(r, 2) for r in range_rates],
            "ms_per_step": round(seconds / n * 1e3, 4), "frac": round(through / HBM_GBPS, 4),
        }
    if not args.no_prefill:
        seconds, flops = prefill_point()
        median = statistics.median(seconds)
        line["prefill"] = {
            "value": round(args.prefill_tokens / median, 1), "tokens": args.prefill_tokens,
            "ms": round(median * 1e3, 3), "frac": round(flops / median / PEAK_FLOPS[args.dtype], 4),
            "runs_ms": [round(s * 1e3, 3) for s in seconds],
        }
    points, fractions, all_runs = {}, {}, {}
    if not args.no_points:
        for batch in (1, 64):
            rates, _, achieved = point(batch, args.context)
            points[f"decode_b{batch}"] = round(statistics.median(rates), 2)
            fractions[f"decode_b{batch}"] = round(achieved / HBM_GBPS, 4)
            all_runs[f"decode_b{batch}"] = [round(r, 2) for r in rates]
    long_contexts = args.long_contexts if args.long_contexts is not None else ("" if args.no_points else "32768")
    for context in [int(c) for c in long_contexts.split(",") if c]:
        rates, _, achieved = point(args.batch, context)
        key = f"decode_b{args.batch}_ctx{context}"
        points[key] = round(statistics.median(rates), 2)
        fractions[key] = round(achieved / HBM_GBPS, 4)
        all_runs[key] = [round(r, 2) for r in rates]
    # other shapes of the family, whole, at the main batch and context: their own bytes and flops
    if not args.no_points and args.layers is None:
        for other in [name for name in args.other_shapes.split(",") if name and name != args.shape]:
            other_shape = SHAPES[other]
            other_layers = other_shape["num_hidden_layers"]
            other_config = Qwen2Config.from_hf_config(dict(other_shape))
            rates, _, achieved = point(args.batch, args.context, other_config, other_layers, f" ({other} shape)")
            key = f"decode_b{args.batch}_{other}"
            points[key] = round(statistics.median(rates), 2)
            fractions[key] = round(achieved / HBM_GBPS, 4)
            all_runs[key] = [round(r, 2) for r in rates]
            if not args.no_prefill:
                seconds, flops = prefill_point(other_config, other_layers, f" ({other} shape)")
                median = statistics.median(seconds)
                key = f"prefill_{args.prefill_tokens}_{other}"
                points[key] = round(args.prefill_tokens / median, 1)
                fractions[key] = round(flops / median / PEAK_FLOPS[args.dtype], 4)
                all_runs[key] = [round(args.prefill_tokens / s, 1) for s in seconds]
    mixed_portions = args.mixed_portions if args.mixed_portions is not None else ("" if args.no_points else "16,64,248")
    portions = [int(c) for c in mixed_portions.split(",") if c]
    if portions:
        say(f"steps of {args.batch} decode tokens beside a prompt portion of {portions}")
        longest = max(portions)
        engine = make_engine(config, args.dtype, args.batch + 1, max(args.context, 64 * longest), args.prefill_tokens)
        took = mixed_steps(engine, config, args.batch, args.context, portions, seed=5)
        del engine
        release()
        line["mixed"] = {"decoding": args.batch, "context": args.context,
                         "ms_per_step": {str(portion): round(s * 1e3, 4) for portion, s in took.items()}}
    if points:
        line["points"] = points
        line["points_frac"] = fractions
        line["points_runs"] = all_runs
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
