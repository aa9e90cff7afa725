"""Small Nokipel configurations for the tests and weights that make faults show.

Random weights of one small scale would hide most faults: every softmax nearly uniform, every gate near one half,
every clamp idle, every router indifferent.  ``make_weights`` draws bolder ones: queries and keys large enough for
peaked attention, projections into the dense unit large enough to reach its limit, gates that open and close, norm
weights away from one, corrections as large as the scores they correct.  Everything is rounded to bfloat16 once, so
that both precisions run the same model.

``exact_router=True`` makes the routers' choices safe from rounding.  The first of the norm's groups of the stream
then holds *markers*: coordinates that are +1 or -1 per token (from the embedding, whose scale is a power of two), to
which no branch writes anything but a common factor (the rows of every output projection that feed them are zero;
the norms' weights on them are 1, so an expert that hands its input on scales them all alike).  A group of +-1, or
of a common multiple of it, norms to +-1 whatever else the stream holds, so a router that reads the markers alone,
through small dyadic weights, gets logits that bfloat16 holds as exactly as float64 does; a last marker that is +1
for every token separates the experts' logits.  Without this a bfloat16 engine and a float64 yardstick would now and
then choose different experts for a token whose two best choice scores lie close, which is no fault of either.  It
needs a configuration whose norm has more than one group; routers that read the whole stream are tested in float32.
"""

from __future__ import annotations

import math

import torch

from polosun_util import Fixed, make_runner, spread  # noqa: F401  (architecture-neutral helpers)

DECAY3 = [0.5, 0.96875, 0.998046875]

MOE_A = {"kind": "moe", "router": {"experts": 7, "identity": 2, "top": 3, "scale": 1.5, "groups": {"count": 3, "keep": 2}},
         "expert": {"ff": 40}, "shared": {"ff": 24}}

# every size differs from its neighbours'; key and value heads of different sizes; a layer without feed-forward, a
# router without groups, identity experts or shared expert; a loop over two layers that runs three times; rotations
# over a part of the head and over all of it; chunks from 5 tokens up
SMALL_A = {
    "architecture": "Nokipel", "vocab": 96, "width": 64, "norm": {"eps": 1e-5, "groups": 4}, "embedding": {"scale": 4.0},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "lightning", "mixer": {"heads": 3, "dim": 16, "vdim": 8, "decay": DECAY3},
         "mlp": {"kind": "dense", "ff": 80, "limit": 0.75}},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 20},
                   "rot": {"base": 100.0, "dims": 8}},
         "mlp": MOE_A},
        {"type": "lightning", "mixer": {"heads": 1, "dim": 8, "vdim": 40, "decay": [0.9375]}, "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 6, "kv_heads": 3, "dim": 8, "vdim": 8, "scale": 0.5, "mask": {"size": 5},
                   "rot": {"base": 7.0, "dims": 8}},
         "mlp": {"kind": "moe", "router": {"experts": 3, "top": 3, "scale": 0.5}, "expert": {"ff": 24}}},
        {"type": "lightning", "mixer": {"heads": 2, "dim": 24, "vdim": 24, "decay": [0.75, 0.9921875]},
         "mlp": {"kind": "dense", "ff": 56, "limit": 2.0}},
    ],
}

# widths that are no multiples of 8, twenty query heads on one key head, a head wider than the matrix-core attention
# takes, a chunk longer than any test sequence, attention without chunks and without rotation, one expert chosen of
# many, a loop from the first layer on, a loop that runs once
SMALL_B = {
    "architecture": "Nokipel", "vocab": 130, "width": 50, "norm": {"eps": 1e-6, "groups": 5}, "embedding": {"scale": 0.5},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 5, "kv_heads": 1, "dim": 12, "vdim": 20, "scale": 0.4, "mask": {"size": 64},
                   "rot": {"base": 10000.0, "dims": 4}},
         "mlp": {"kind": "moe", "router": {"experts": 10, "identity": 5, "top": 4, "scale": 2.0, "groups": {"count": 5, "keep": 2}},
                 "expert": {"ff": 30}, "shared": {"ff": 22}}},
        {"type": "lightning", "mixer": {"heads": 5, "dim": 8, "vdim": 16, "decay": [0.25, 0.5, 0.75, 0.875, 0.999]},
         "mlp": {"kind": "dense", "ff": 72, "limit": 1.0}},
        {"type": "attention",
         "mixer": {"heads": 20, "kv_heads": 1, "dim": 64, "vdim": 32, "scale": 0.06, "mask": {"size": 1000}},
         "mlp": {"kind": "moe", "router": {"experts": 12, "top": 1, "scale": 1.0}, "expert": {"ff": 18}, "shared": {"ff": 8}}},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 136, "vdim": 8, "scale": 0.05, "rot": {"base": 30.0, "dims": 136}},
         "mlp": None},
    ],
}

SMALL = {"A": SMALL_A, "B": SMALL_B}


def single(layer: dict, width: int = 32, vocab: int = 50, groups: int = 2, loop: dict | None = None) -> dict:
    """A model of one layer: a mechanism alone."""
    out = {"architecture": "Nokipel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6, "groups": groups},
           "embedding": {"scale": 0.5}, "layers": [layer]}
    if loop:
        out["loop"] = loop
    return out


def markers_of(raw: dict) -> int:
    """How many stream coordinates the markers take: the norm's first group."""
    return raw["width"] // raw["norm"].get("groups", 1)


def make_weights(raw: dict, seed: int, sharp: float = 1.0, exact_router: bool = False) -> dict[str, torch.Tensor]:
    """Float32 tensors (bfloat16-representable values) for every name the configuration's model expects."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors

    expected = expected_tensors(config_from_dict(raw).model_spec())
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        if spec.optional:
            continue
        shape = tuple(spec.shape)
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        fan_in = shape[-1] if len(shape) >= 2 else 1
        if leaf in ("norm1", "norm2", "mix.norm") or name == "final.norm":
            t = 0.6 + 0.8 * torch.rand(shape, generator=g)
        elif leaf == "mlp.correction":
            t = torch.rand(shape, generator=g) * 0.5 - 0.3                  # some choice scores are negative
        elif leaf.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf in ("mix.q", "mix.k"):
            t = torch.randn(shape, generator=g) * (2.0 * sharp / math.sqrt(fan_in))
        elif leaf in ("mix.g", "mlp.shared.sg"):
            t = torch.randn(shape, generator=g) * (3.0 / math.sqrt(fan_in))
        elif leaf.endswith(".gate") or leaf.endswith(".up"):
            t = torch.randn(shape, generator=g) * (2.0 / math.sqrt(fan_in))   # reaches the limits now and then
        elif leaf == "mlp.router":
            t = torch.randn(shape, generator=g) * (4.0 / math.sqrt(fan_in))
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / math.sqrt(fan_in))
        out[name] = t
    if exact_router:
        m = markers_of(raw)
        scale = float(raw.get("embedding", {}).get("scale", 1.0))
        if raw["norm"].get("groups", 1) < 2 or m < 3 or math.log2(scale) != int(math.log2(scale)):
            raise ValueError("markers need a norm of several groups, three coordinates and an embedding scale that is a power of two")
        vocab = out["embed"].shape[0]
        marks = torch.randint(0, 2, (vocab, m), generator=g).float() * 2.0 - 1.0
        marks[:, m - 1] = 1.0
        out["embed"][:, :m] = marks / scale
        for name in list(out):
            leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
            if leaf == "mix.o" or leaf.endswith(".down"):
                out[name][:m] = 0.0                                       # no branch writes to the markers ...
            if leaf in ("norm1", "norm2"):
                out[name][:m] = 1.0                                       # ... and a handed-on row scales them alike
            if leaf == "mlp.router":
                outputs = out[name].shape[0]
                router = torch.zeros_like(out[name])
                router[:, : m - 1] = torch.randint(-2, 3, (outputs, m - 1), generator=g).float() * 0.5
                # no two outputs' logits are equal: the other markers move a logit in steps of one, this one by
                # less than that in all
                steps = 2 << max(outputs - 1, 1).bit_length()
                router[:, m - 1] = torch.arange(outputs).float() / steps
                out[name] = router
    return {name: t.to(torch.bfloat16).float() for name, t in out.items()}
