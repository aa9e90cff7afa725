"""Position encodings.

``RotaryHalf``: rotary encoding with half-split pairing (element ``i`` rotates
with ``i + R/2`` for the first ``R = rotary_dim`` dimensions of a head, all of
them unless told otherwise; the rest pass through), tables as in the reference's ``build_rope_cache``
(src/cloud_engine/attention.py:60-67): ``inv_freq_j = 1 / theta^(2j/D)``,
``angle[p, j] = p * inv_freq_j`` in float32, then cos and sin.  The reference
fixes the table length at 32768 (src/cloud_engine/model.py:188-192); here it is
``max_position``.  Tables are computed once on the CPU in float32 (so they do
not depend on the GPU's transcendental functions) and shared by every layer
with the same constants.

Two extensions that a configuration may ask for.  ``scaling=(factor, original, fast, slow)`` stretches the slow
pairs for contexts beyond the ``original`` length the frequencies were made for: with
``turn(t) = R ln(original / (2 pi t)) / (2 ln theta)`` the pair index that makes ``t`` turns over that length,
``lo = max(floor(turn(fast)), 0)``, ``hi = min(ceil(turn(slow)), R - 1)`` and
``ramp_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1)``, pair j turns at
``inv_freq_j * (1 - ramp_j) + inv_freq_j / factor * ramp_j``, and cos and sin are both multiplied by
``0.1 ln(factor) + 1``.  ``scaling=(factor,)`` alone divides every frequency by the factor and leaves cos and sin as
they are.  ``max_position=None`` is a model without a longest position: the tables then grow as
positions are asked for (``tables(device, upto)``), in powers of two.
"""

from __future__ import annotations

import math

import torch

from .base import Part, register_part

_TABLES: dict[tuple, tuple[torch.Tensor, torch.Tensor]] = {}


class RotaryHalf(Part):
    graph_safe = True
    rotates = True
    pairing = "halves"

    UNBOUNDED = 1 << 30   # what ``max_position`` reads as where the model names no longest position
    FIRST_ROWS = 4096     # the smallest table of a model without one

    def __init__(self, head_dim: int, theta: float, max_position: int | None, rotary_dim: int | None = None,
                 scaling: tuple | None = None) -> None:
        rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if head_dim <= 0 or rotary_dim <= 0 or rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError(f"rotary_dim must be even, positive and at most the head size {head_dim}, got {rotary_dim}")
        if not theta > 0 or (max_position is not None and max_position <= 0):
            raise ValueError("rotary theta and max_position must be positive")
        if scaling is not None:
            scaling = tuple(float(v) for v in scaling)
            if len(scaling) not in (1, 4) or not all(v > 0 for v in scaling) or (len(scaling) == 4 and theta == 1.0):
                raise ValueError(f"scaling is (factor,) or (factor, original, fast, slow), all positive, got {scaling}")
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.grows = max_position is None
        self.max_position = self.UNBOUNDED if max_position is None else max_position
        self.scaling = scaling

    def inv_freq(self) -> tuple[torch.Tensor, float]:
        """float32 frequencies of the pairs, and the factor on cos and sin."""
        inv_freq = 1.0 / (
            self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim)
        )
        if self.scaling is None:
            return inv_freq, 1.0
        if len(self.scaling) == 1:
            return inv_freq / self.scaling[0], 1.0
        factor, original, fast, slow = self.scaling
        turn = lambda t: self.rotary_dim * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(turn(fast)), 0)
        hi = min(math.ceil(turn(slow)), self.rotary_dim - 1)
        pair = torch.arange(self.rotary_dim // 2, dtype=torch.float32)
        ramp = ((pair - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return inv_freq / factor * ramp + inv_freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0

    def tables(self, device: torch.device, upto: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """(cos, sin), each float32 ``[positions, rotary_dim/2]`` (the two halves of the reference's table are equal,
        so one half is kept).  ``positions`` is ``max_position``, or, for a model without one, the power of two that
        holds position ``upto - 1`` (what was made for fewer is made anew; angles are position times frequency in
        float32 either way, so a position's row does not depend on the table's length)."""
        rows = self.max_position
        if self.grows:
            rows = max(self.FIRST_ROWS, 1 << max(0, (upto or 1) - 1).bit_length())
        key = (self.rotary_dim, self.theta, self.scaling, self.grows, str(device))
        if not self.grows:
            key += (rows,)
        kept = _TABLES.get(key)
        if kept is None or kept[0].shape[0] < rows:
            inv_freq, gain = self.inv_freq()
            positions = torch.arange(rows, dtype=torch.float32)
            angles = positions[:, None] * inv_freq[None, :]
            kept = _TABLES[key] = ((angles.cos() * gain).to(device).contiguous(), (angles.sin() * gain).to(device).contiguous())
        return kept


class RotaryPairs(RotaryHalf):
    """The same angles, with neighbours as partners: of the first ``rotary_dim`` numbers of a head, numbers
    ``2i`` and ``2i + 1`` turn together by ``p * theta^(-2i / rotary_dim)``,
    ``(u, v) -> (u cos - v sin, v cos + u sin)``.  The tables are those of the half-split pairing (an angle does
    not know its partners); the kernel that turns the heads is told the pairing."""

    pairing = "neighbours"


class NoPosition(Part):
    graph_safe = True
    """Keys and queries enter the mixer as projected."""

    rotates = False

    def __init__(self, head_dim: int = 0, max_position: int = 1) -> None:
        self.head_dim = head_dim
        self.rotary_dim = 0
        self.max_position = max_position

    def tables(self, device: torch.device, upto: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        key = ("none", max(self.head_dim, 2), str(device))
        if key not in _TABLES:
            zeros = torch.zeros((1, max(self.head_dim, 2) // 2), dtype=torch.float32, device=device)
            _TABLES[key] = (zeros, zeros)
        return _TABLES[key]


register_part("position", "rotary_half", RotaryHalf)
register_part("position", "rotary_pairs", RotaryPairs)
register_part("position", "none", NoPosition)
