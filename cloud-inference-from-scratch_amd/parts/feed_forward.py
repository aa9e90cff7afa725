"""Gated feed-forward (SwiGLU): ``down(act(gate(x)) * up(x))`` without biases.

Reference: ``Qwen2MLP`` (src/cloud_engine/model.py:86-100).  Gate and up are
one fused product here, the activation and the multiply one kernel.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, register_part
from .linear import linear


class GatedMLP(Part):
    graph_safe = True
    adds_to_residual = True
    takes_scaled_rows = True  # its first product applies the scale of rows that come without it
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")) -> None:
        if activation != "silu":
            raise ValueError(f"gated feed-forward runs silu only, got {activation!r}")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.names = tuple(names)  # what the checkpoint calls the gate, up and down weights under the part's prefix

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        gate, up, down = self.names
        return {
            prefix + gate: TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + up: TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + down: TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[prefix + gate], tensors[prefix + up]], dim=0).contiguous()
        self.w_down = tensors[prefix + down].contiguous()

    def warm_up(self, rows: int) -> None:
        self.forward(torch.zeros((rows, self.hidden_size), dtype=self.w_down.dtype, device=self.w_down.device))

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        return linear(linear(x, self.w_gate_up, epilogue="silu"), self.w_down, into=residual)


class ClampedGatedMLP(Part):
    """A dense gated feed-forward whose unit bounds its inputs: ``g = min(W_gate x, limit)``,
    ``u = clamp(W_up x, -limit, limit)``, ``y = W_down (g * sigmoid(alpha g) * (u + offset))``.  ``limit``, ``alpha``
    and ``offset`` are parameters (``limit=None``: unbounded; ``alpha=1, offset=0`` is ``silu(g) * u``); the unit is
    computed in float32 from the product's rows.  ``cubic`` puts ``g + cubic * g^3`` inside the sigmoid:
    ``alpha = 2 sqrt(2 / pi)`` with ``cubic = 0.044715`` is the tanh form of gelu on the gate (``GELU_TANH``)."""

    graph_safe = True
    GELU_TANH = dict(alpha=2.0 * (2.0 / 3.141592653589793) ** 0.5, cubic=0.044715, offset=0.0)

    def __init__(self, hidden_size: int, intermediate_size: int, limit: Optional[float] = None, alpha: float = 1.0,
                 offset: float = 0.0, names: tuple[str, str, str] = ("gate", "up", "down"), cubic: float = 0.0) -> None:
        if min(hidden_size, intermediate_size) < 1 or (limit is not None and not limit > 0):
            raise ValueError("sizes and the limit must be positive")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.limit = float("inf") if limit is None else float(limit)
        self.alpha, self.offset, self.cubic = float(alpha), float(offset), float(cubic)
        self.names = tuple(names)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        gate, up, down = self.names
        return {
            prefix + gate: TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + up: TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + down: TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[prefix + gate], tensors[prefix + up]], dim=0).contiguous()
        self.w_down = tensors[prefix + down].contiguous()

    def warm_up(self, rows: int) -> None:
        self.forward(torch.zeros((rows, self.hidden_size), dtype=self.w_down.dtype, device=self.w_down.device))

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        hidden = ops.clamped_glu(linear(x, self.w_gate_up), self.limit, self.alpha, self.offset, self.cubic)
        return linear(hidden, self.w_down)


class NoFeedForward(Part):
    """A layer without a feed-forward: no tensors, and ``forward`` gives nothing to add."""

    graph_safe = True

    def __init__(self, hidden_size: int = 0) -> None:
        self.hidden_size = hidden_size

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        return None


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "clamped_gated_mlp", ClampedGatedMLP)
register_part("feed_forward", "none", NoFeedForward)
