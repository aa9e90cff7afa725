"""A feed-forward of many small gated experts, of which every token uses the few that a router scores highest,
beside an expert that every token uses.

    z = W_router x (float32),  s = sigmoid(z),  the ``top`` largest chosen, their scores kept as they are
    y = sum_chosen expert_e(s_e * x) + shared(x)
    expert(v) = W_down (g * sigmoid(alpha g) * (u + offset)),  g = min(W_gate v, limit),  u = clamp(W_up v, -limit, limit)

The score multiplies the expert's input, and since the unit is not linear it stays there.  ``alpha``, ``offset``,
the limits and all sizes are parameters; the shared expert is optional and has its own size and limit.

What a design may change, each a parameter: the scores (``scoring="softmax"``: over all router outputs), a
``correction`` tensor that is added to the scores for the choice only, groups of neighbouring outputs of which only
the best ``keep`` can be chosen (``groups=(count, keep)``; a group counts by its largest corrected score),
``normalize`` (the chosen scores divided by their sum + 1e-20) and ``route_scale``, ``identity`` router outputs behind
the experts that hand the token's row on instead of running weights, ``weight_on="output"`` (the score multiplies
the expert's output row, in the kernel that sums a token's rows), experts and a shared expert without limits
(``None``), and ``shared_gate`` (the shared expert's output times ``sigmoid(w_sg . x)``, one number per token).

The router's product has float32 sums and a float32 result; scores, choice and order by expert are made on the device
(``ops.experts_route``), so nothing of a step waits for the host and a step can be captured.  The experts' products
run per tile of rows of one expert (``ops.experts_forward``: bfloat16 on the matrix cores, float32 as plain
multiply-adds in order); the shared expert is two ordinary products with the unit between them.  What comes back is a
``SummedBranch``: the shared expert's rows and one float32 row per (token, choice), which the kernel that adds the
branch sums in a fixed order.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, register_part
from .linear import SummedBranch, linear


class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, experts: int, top: int, expert_ff: int, expert_limit: float,
                 shared_ff: Optional[int] = None, shared_limit: Optional[float] = None, alpha: float = 1.702,
                 offset: float = 1.0, scoring: str = "sigmoid", correction: bool = False,
                 groups: Optional[tuple] = None, identity: int = 0, normalize: bool = False, route_scale: float = 1.0,
                 weight_on: str = "input", shared_gate: bool = False) -> None:
        for name, value in (("hidden_size", hidden_size), ("experts", experts), ("top", top), ("expert_ff", expert_ff)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        if isinstance(identity, bool) or not isinstance(identity, int) or identity < 0:
            raise ValueError(f"identity must be a count, got {identity!r}")
        outputs = experts + identity
        if top > outputs or outputs > ops.MAX_EXPERTS:
            raise ValueError(f"{top} of {outputs} router outputs: at most all of them, and at most {ops.MAX_EXPERTS}")
        unbounded = lambda limit: limit is None or limit == float("inf")
        if not (unbounded(expert_limit) or expert_limit > 0):
            raise ValueError("limits must be positive")
        if shared_ff is not None and not (shared_ff >= 1 and (unbounded(shared_limit) or shared_limit > 0)):
            raise ValueError("a shared expert needs a positive size, and its limit must be positive")
        if scoring not in ("sigmoid", "softmax") or weight_on not in ("input", "output"):
            raise ValueError(f"scoring {scoring!r} / weight_on {weight_on!r}: sigmoid or softmax, input or output")
        if identity and weight_on != "output":
            raise ValueError("experts that hand their input on take their weight on the output")
        if groups is not None:
            count, keep = (int(v) for v in groups)
            if not (1 <= keep <= count <= ops.MAX_EXPERT_GROUPS and outputs % count == 0 and top <= keep * (outputs // count)):
                raise ValueError(f"{count} groups of which {keep} are kept do not fit {top} of {outputs} router outputs")
            groups = (count, keep)
        if shared_gate and shared_ff is None:
            raise ValueError("a gate on the shared expert needs a shared expert")
        self.hidden_size, self.experts, self.top, self.expert_ff = hidden_size, experts, top, expert_ff
        self.expert_limit = float("inf") if unbounded(expert_limit) else float(expert_limit)
        self.shared_ff = shared_ff
        self.shared_limit = None if shared_ff is None else float("inf") if unbounded(shared_limit) else float(shared_limit)
        self.alpha, self.offset = float(alpha), float(offset)
        self.scoring, self.has_correction, self.groups, self.identity = scoring, bool(correction), groups, identity
        self.normalize, self.route_scale, self.weight_on = bool(normalize), float(route_scale), weight_on
        self.shared_gate = bool(shared_gate)
        self.outputs = outputs

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        width, ff = self.hidden_size, self.expert_ff
        out = {prefix + "router": TensorSpec((self.outputs, width))}
        if self.has_correction:
            out[prefix + "correction"] = TensorSpec((self.outputs,), keeps_float32=True)
        if self.shared_gate:
            out[prefix + "shared.sg"] = TensorSpec((1, width))
        for e in range(self.experts):
            out[f"{prefix}e{e}.gate"] = TensorSpec((ff, width))
            out[f"{prefix}e{e}.up"] = TensorSpec((ff, width))
            out[f"{prefix}e{e}.down"] = TensorSpec((width, ff))
        if self.shared_ff is not None:
            out[prefix + "shared.gate"] = TensorSpec((self.shared_ff, width))
            out[prefix + "shared.up"] = TensorSpec((self.shared_ff, width))
            out[prefix + "shared.down"] = TensorSpec((width, self.shared_ff))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.w_router = tensors[prefix + "router"].contiguous()
        self.correction = tensors[prefix + "correction"].float().contiguous() if self.has_correction else None
        self.w_shared_gate = None
        if self.shared_gate:
            # (eight rows of which the first is the gate's: the products' result rows stay 16-byte aligned)
            w_sg = tensors[prefix + "shared.sg"]
            self.w_shared_gate = torch.cat([w_sg, w_sg.new_zeros((7, self.hidden_size))], dim=0).contiguous()
        self.w_gate_up = torch.stack([torch.cat([tensors[f"{prefix}e{e}.gate"], tensors[f"{prefix}e{e}.up"]], dim=0)
                                      for e in range(self.experts)]).contiguous()
        self.w_down = torch.stack([tensors[f"{prefix}e{e}.down"] for e in range(self.experts)]).contiguous()
        self.w_shared_gate_up = self.w_shared_down = None
        if self.shared_ff is not None:
            self.w_shared_gate_up = torch.cat([tensors[prefix + "shared.gate"], tensors[prefix + "shared.up"]], dim=0).contiguous()
            self.w_shared_down = tensors[prefix + "shared.down"].contiguous()
        # the matrix cores take bfloat16 rows whose widths are multiples of 8
        self.mfma = dtype == torch.bfloat16 and self.hidden_size % 8 == 0 and self.expert_ff % 8 == 0

    def warm_up(self, rows: int) -> None:
        if self.shared_ff is not None:
            blank = lambda width: torch.zeros((rows, width), dtype=self.w_down.dtype, device=self.w_down.device)
            linear(blank(self.hidden_size), self.w_shared_gate_up)
            linear(blank(self.shared_ff), self.w_shared_down)

    def tile_rows(self, tokens: int) -> int:
        """Rows of one expert a workgroup takes: as many as an expert gets on average, within what the form has."""
        if not self.mfma:
            return 16
        mean = tokens * self.top / self.outputs
        return 128 if mean > 48 else 64 if mean > 32 else 32 if mean > 16 else 16

    def forward(self, x: torch.Tensor):
        tokens = x.shape[0]
        logits = linear(x, self.w_router, out_dtype=torch.float32)
        route = ops.experts_route(logits, self.top, self.tile_rows(tokens), real=self.experts, scoring=self.scoring,
                                  correction=self.correction, groups=self.groups, normalize=self.normalize,
                                  scale=self.route_scale)
        on_input = self.weight_on == "input"
        parts = ops.experts_forward(x, route, self.w_gate_up, self.w_down, self.expert_limit, self.alpha, self.offset,
                                    mfma=self.mfma, weight_input=on_input)
        shared = gate = None
        if self.shared_ff is not None:
            hidden = ops.clamped_glu(linear(x, self.w_shared_gate_up), self.shared_limit, self.alpha, self.offset)
            shared = linear(hidden, self.w_shared_down)
            if self.w_shared_gate is not None:
                gate = linear(x, self.w_shared_gate, out_dtype=torch.float32)[:, 0]  # (the norm kernel strides over the rows)
        weights = None if on_input else route.pair_weight.view(tokens, self.top)
        return SummedBranch(shared, parts, weights=weights, main_gate=gate)


register_part("feed_forward", "routed_experts", RoutedExperts)
