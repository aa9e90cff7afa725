"""Small Senuvik configurations for the tests and weights that make faults show.

Random weights of one small scale would hide most faults: every softmax nearly uniform, every gate near one half,
every decay the same, every router indifferent.  ``make_weights`` draws bolder ones: queries and keys large enough for
peaked attention, sinks that take a share of the softmax, decays spread over their range, gates that open and close,
norm weights and scales per channel away from one.  Everything is rounded to bfloat16 once, so that both precisions
run the same model.

``exact_router=True`` makes the routers' choices safe from rounding.  The first ``MARKERS`` coordinates of the stream
then hold *markers*: +1 or -1 per token (from the embedding), to which no branch writes (the rows of every output
projection that feed them are zero, and a zero stays zero under the norm on the branch's output).  A norm of the
stream multiplies them all by one factor, so a router that reads the markers alone, through small dyadic weights,
ranks its outputs in bfloat16 as it does in float64; a last marker that is +1 for every token separates the outputs'
logits.  Without this a bfloat16 engine and a float64 yardstick would now and then choose different experts for a
token whose two best logits lie close, which is no fault of either.  Routers that read the whole stream are tested in
float32.
"""

from __future__ import annotations

import math

import torch

from polosun_util import Fixed, make_runner, spread  # noqa: F401  (architecture-neutral helpers)

MARKERS = 6
YARN = {"factor": 4.0, "fast": 16.0, "original": 64, "slow": 1.0}

MOE_A = {"kind": "moe", "router": {"experts": 6, "top": 2}, "expert": {"ff": 24}, "shared": {"ff": 16}}

# every size differs from its neighbours'; key and value heads of different sizes; a layer without feed-forward, a
# router without shared expert that takes all its experts; a layer that reads another's keys under a mask of its own;
# rotations over a part of the head; a state-space layer of one head, one group, one tap and one norm group
SMALL_A = {
    "architecture": "Senuvik", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 9, "keep_first": 3},
                   "rot": {"base": 100.0, "dims": 8, "scaling": {"factor": 2.0}}},
         "mlp": {"kind": "dense", "ff": 80}},
        {"type": "mamba2", "mixer": {"heads": 4, "vdim": 8, "state": 12, "groups": 2, "conv": 4, "norm_groups": 2},
         "mlp": MOE_A},
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.35, "softcap": 5.0,
                            "rot": {"base": 1000.0, "dims": 8, "scaling": YARN}},
                   "right": {"heads": 2, "dim": 12}, "left_scale": 0.7, "right_scale": 0.4},
         "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "kv_from": 0,
                   "mask": {"size": 20, "keep_first": 0},
                   "rot": {"base": 100.0, "dims": 8, "scaling": {"factor": 2.0}}},
         "mlp": {"kind": "moe", "router": {"experts": 3, "top": 3}, "expert": {"ff": 24}}},
        {"type": "mamba2", "mixer": {"heads": 1, "vdim": 40, "state": 5, "groups": 1, "conv": 1, "norm_groups": 1},
         "mlp": {"kind": "dense", "ff": 56}},
    ],
}

# a width that is no multiple of 8, twenty query heads on one key head, a head wider than the matrix-core attention
# takes, a window longer than any test sequence, more kept first tokens than the window holds, a reader whose window is
# shorter than the writer's, one expert chosen of many, the parallel layer first
SMALL_B = {
    "architecture": "Senuvik", "vocab": 130, "width": 50, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 5, "kv_heads": 5, "dim": 12, "vdim": 20, "scale": 0.4, "softcap": 30.0,
                            "rot": {"base": 50.0, "dims": 12}},
                   "right": {"heads": 5, "dim": 8}, "left_scale": 1.25, "right_scale": 1.0},
         "mlp": {"kind": "moe", "router": {"experts": 12, "top": 1}, "expert": {"ff": 18}, "shared": {"ff": 8}}},
        {"type": "attention",
         "mixer": {"heads": 20, "kv_heads": 1, "dim": 64, "vdim": 32, "scale": 0.06, "mask": {"size": 1000, "keep_first": 0},
                   "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 1.0}}},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "mamba2", "mixer": {"heads": 6, "vdim": 16, "state": 64, "groups": 3, "conv": 2, "norm_groups": 3},
         "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 20, "kv_heads": 1, "dim": 64, "vdim": 32, "scale": 0.1, "kv_from": 1,
                   "mask": {"size": 7, "keep_first": 10},
                   "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 1.0}}},
         "mlp": {"kind": "moe", "router": {"experts": 5, "top": 4}, "expert": {"ff": 30}, "shared": {"ff": 22}}},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 2, "dim": 136, "vdim": 8, "scale": 0.05, "mask": {"size": 33, "keep_first": 5},
                   "rot": {"base": 30.0, "dims": 136, "scaling": {"factor": 8.0}}},
         "mlp": None},
    ],
}

SMALL = {"A": SMALL_A, "B": SMALL_B}


def single(layer: dict, width: int = 32, vocab: int = 50, before: dict | None = None) -> dict:
    """A model of one layer: a mechanism alone (``before``: a layer in front of it, for one that reads another's keys)."""
    return {"architecture": "Senuvik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "layers": ([before] if before else []) + [layer]}


def make_weights(raw: dict, seed: int, sharp: float = 1.0, exact_router: bool = False, rank: int = 8) -> dict[str, torch.Tensor]:
    """Float32 tensors (bfloat16-representable values) for every name the configuration's model expects."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors

    expected = expected_tensors(config_from_dict(raw).model_spec())
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        if spec.optional:
            continue
        shape = tuple(rank if size is None else size for size in spec.shape)
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        last = leaf.rsplit(".", 1)[-1]
        fan_in = shape[-1] if len(shape) >= 2 else 1
        normal = lambda scale: torch.randn(shape, generator=g) * scale
        if last in ("norm1", "norm2", "norm1b", "norm2b", "ls1", "ls2", "norm") or name == "final.norm":
            t = 0.6 + 0.8 * torch.rand(shape, generator=g)
        elif leaf.endswith(".b") and "conv" not in leaf:
            t = normal(0.5)
        elif last in ("q", "k") and "right" not in leaf:
            t = normal(2.0 * sharp / math.sqrt(fan_in))
        elif last == "sink":
            t = normal(1.5)
        elif leaf.endswith("left.g") or leaf == "mlp.shared.sg":
            t = normal(3.0 / math.sqrt(fan_in))
        elif last in ("gate", "up"):
            t = normal(2.0 / math.sqrt(fan_in))
        elif leaf == "mlp.router":
            t = normal(4.0 / math.sqrt(fan_in))
        elif leaf == "mix.conv":
            t = normal(0.6)
        elif leaf == "mix.conv.b":
            t = normal(0.3)
        elif leaf == "mix.dt_bias":
            t = torch.linspace(-3.0, 1.0, shape[0])[torch.randperm(shape[0], generator=g)]
        elif leaf == "mix.A_log":
            t = torch.linspace(-2.0, 1.0, shape[0])[torch.randperm(shape[0], generator=g)]
        elif leaf == "mix.D":
            t = 0.5 + torch.rand(shape, generator=g)
        elif ".mu." in leaf:
            t = torch.rand(shape, generator=g)
        elif last == "w0":
            t = torch.linspace(-5.0, 0.5, shape[0])[torch.randperm(shape[0], generator=g)]
        elif last in ("w1", "w2"):
            t = normal(1.5 / math.sqrt(fan_in))
        elif last == "u":
            t = normal(0.5)
        elif name == "embed":
            t = normal(1.0)
        else:
            t = normal(1.0 / math.sqrt(fan_in))
        out[name] = t
    if exact_router:
        m = MARKERS
        vocab = out["embed"].shape[0]
        marks = torch.randint(0, 2, (vocab, m), generator=g).float() * 2.0 - 1.0
        marks[:, m - 1] = 1.0
        out["embed"][:, :m] = marks
        for name in list(out):
            last = name.rsplit(".", 1)[-1]
            if last in ("o", "down"):
                out[name][:m] = 0.0                                       # no branch writes to the markers
            if last in ("norm1", "norm2"):
                out[name][:m] = 1.0
            if name.endswith("mlp.router"):
                outputs = out[name].shape[0]
                router = torch.zeros_like(out[name])
                router[:, : m - 1] = torch.randint(-2, 3, (outputs, m - 1), generator=g).float() * 0.5
                # no two outputs' logits are equal: the other markers move a logit in steps of one half of the common
                # factor, this one by less than that in all
                steps = 4 << max(outputs - 1, 1).bit_length()
                router[:, m - 1] = torch.arange(outputs).float() / steps
                out[name] = router
    return {name: t.to(torch.bfloat16).float() for name, t in out.items()}
