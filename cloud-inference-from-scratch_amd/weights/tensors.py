"""What a part says about each tensor it wants from a checkpoint."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class TensorSpec:
    """``shape`` as stored.  ``init`` tells the random-weights mode how to fill
    it: ``"normal"`` is N(0, std), ``"norm"`` is 1 + N(0, std).  ``kind`` is
    ``"float"`` (runs in the engine's dtype) or ``"int"`` (kept as int32).
    ``keeps_float32``: a small vector (norm weight) that stays in 32-bit when the
    file stores it so, whatever the engine's dtype.  ``optional``: a tensor that a checkpoint may hold although
    this model does not read it; it is neither missed nor called unexpected.  An entry of ``shape`` may be ``None``:
    a size that only the checkpoint knows (the part reads it off the tensor it is bound to); ``drawn`` is then the
    shape that the random-weights mode makes."""

    shape: tuple
    init: str = "normal"
    kind: str = "float"
    keeps_float32: bool = False
    optional: bool = False
    drawn: tuple | None = None

    def fits(self, stored: tuple) -> bool:
        """Whether a stored tensor's shape is this one (a free size fits any)."""
        return len(stored) == len(self.shape) and all(want is None or want == have
                                                      for want, have in zip(self.shape, stored))

    @property
    def random_shape(self) -> tuple:
        if self.drawn is not None:
            return tuple(self.drawn)
        if any(size is None for size in self.shape):
            raise ValueError(f"a tensor of shape {self.shape} needs a shape to be drawn at")
        return tuple(self.shape)
