"""Two mixers side by side: both read the same rows, and the layer's branch is a weighted sum of their outputs,
``left_scale * left(x) + right_scale * right(x)``.  The two are parts of any kind (an attention beside a recurrent
memory, say), built from their own specs under the tensor prefixes ``left.`` and ``right.``; the cache unit of the
layer holds the cells of both, the left one's first.  The sum itself is left to whoever adds the branch to the
stream (a :class:`~cie_amd.parts.linear.WeightedPair`), so that it costs no kernel of its own.
"""

from __future__ import annotations

from typing import Any

import torch

from ..config.specs import PartSpec
from ..weights.tensors import TensorSpec
from .base import Part, build_part, register_part
from .linear import WeightedPair


def _cells(need: Any) -> tuple:
    if need is None:
        return ()
    return tuple(need) if isinstance(need, (tuple, list)) else (need,)


class ParallelMixers(Part):
    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 names: tuple[str, str] = ("left", "right")) -> None:
        self.left = build_part("mixer", left)
        self.right = build_part("mixer", right)
        self.scales = (float(left_scale), float(right_scale))
        self.names = tuple(names)
        self._left_cells = len(_cells(self.left.cache_need()))
        self._right_cells = len(_cells(self.right.cache_need()))

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    def cache_need(self) -> Any:
        cells = _cells(self.left.cache_need()) + _cells(self.right.cache_need())
        return cells if len(cells) > 1 else (cells[0] if cells else None)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out = dict(self.left.expected_tensors(f"{prefix}{self.names[0]}."))
        out.update(self.right.expected_tensors(f"{prefix}{self.names[1]}."))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.left.bind(tensors, f"{prefix}{self.names[0]}.", dtype, device)
        self.right.bind(tensors, f"{prefix}{self.names[1]}.", dtype, device)

    def warm_up(self, rows: int) -> None:
        for part in (self.left, self.right):
            warm = getattr(part, "warm_up", None)
            if warm is not None:
                warm(rows)

    @staticmethod
    def _view_of(cells: tuple, count: int) -> Any:
        return None if count == 0 else cells[0] if count == 1 else cells

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> WeightedPair:
        cells = tuple(view) if isinstance(view, (tuple, list)) else ((view,) if view is not None else ())
        left_view = self._view_of(cells[: self._left_cells], self._left_cells)
        right_view = self._view_of(cells[self._left_cells:], self._right_cells)
        first = self.left.forward(x, batch, left_view, writes)
        second = self.right.forward(x, batch, right_view, writes)
        return WeightedPair(first, second, self.scales)


register_part("mixer", "parallel_mixers", ParallelMixers)
