"""Arrangement of a layer's parts.

``PreNormBlock``: the reference's decoder layer (src/cloud_engine/model.py:211-220)
``h += mixer(norm1(h)); h += feed_forward(norm2(h))``.  The residual stream is
float32; a branch's output is added inside the next norm kernel, so the block
returns the feed-forward output as ``pending`` instead of adding it.  A part
that can add its output into the residual itself (the fused decode products do)
returns a ``RowSumsq`` or an ``Added`` instead, and the next norm then runs its
cheaper form or rides along with the product behind it (``parts/linear.py``).

``BranchNormBlock``: the sublayers read the stream itself and their outputs are normed before they are added:
``h += norm1(mixer(h)); h += norm2(feed_forward(h))``.

``SandwichNormBlock``: a norm in front of every sublayer and one on its output, which is then scaled per channel:
``h += s1 * norm1_out(mixer(norm1(h))); h += s2 * norm2_out(feed_forward(norm2(h)))``.

``ParallelDepthBlock``: both branches read the same stream, and the next layer reads a weighted average of what
the embedding and all layers so far left (below).
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Optional

import torch

from ..config.specs import LayerSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import build_part, register_part
from .linear import Added, RawRows, RowSumsq, StreamRows, WeightedPair


class PreNormBlock:
    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        self.norm2 = build_part("norm", spec.norm2)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)
        # a layer without feed-forward has no second norm (a checkpoint that holds one all the same is accepted)
        self.has_feed_forward = spec.feed_forward.kind != "none"

    def _parts(self):
        if not self.has_feed_forward:
            return (("norm1", self.norm1), ("mixer", self.mixer))
        return (("norm1", self.norm1), ("mixer", self.mixer), ("norm2", self.norm2),
                ("feed_forward", self.feed_forward))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out: dict[str, TensorSpec] = {}
        for role, part in self._parts():
            out.update(part.expected_tensors(f"{prefix}{self.spec.name_of(role)}."))
        if not self.has_feed_forward:
            for name, spec in self.norm2.expected_tensors(f"{prefix}{self.spec.name_of('norm2')}.").items():
                out[name] = replace(spec, optional=True)
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        self.dtype = dtype
        for role, part in self._parts():
            part.bind(tensors, f"{prefix}{self.spec.name_of(role)}.", dtype, device)

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._parts())

    def warm_up(self, rows: int) -> None:
        for _, part in self._parts():
            warm = getattr(part, "warm_up", None)
            if warm is not None:
                warm(rows)

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], batch, view,
                writes: bool = True, plus: Optional[torch.Tensor] = None) -> tuple[torch.Tensor, torch.Tensor]:
        """``plus``: float32 rows that join the stream in front of this layer (behind what is pending).  A first
        norm that says ``takes_plus`` adds them in its own kernel; for any other they are added here."""
        if plus is not None:
            if getattr(self.norm1, "takes_plus", False):
                x = self.norm1.forward(residual, pending, self.dtype, plus=plus)
                return self._behind_first_norm(x, residual, batch, view, writes)
            x = normalise(self.norm1, residual, pending, self.dtype)  # (the pending branch joins the stream)
            residual.add_(plus)
            pending = None
        if ((pending is None or isinstance(pending, Added)) and getattr(self.mixer, "takes_raw_rows", False)
                and getattr(self.norm1, "folds_into_products", False) and RawRows.fits(residual, self.dtype)):
            # a few rows, the stream complete: the mixer's first product makes the norm itself (a kernel less)
            x = RawRows(residual, self.norm1, self.dtype)
        else:
            x = normalise(self.norm1, residual, pending, self.dtype)
        return self._behind_first_norm(x, residual, batch, view, writes)

    def _behind_first_norm(self, x, residual: torch.Tensor, batch, view, writes: bool):
        extra = {"residual": residual} if getattr(self.mixer, "adds_to_residual", False) else {}
        if (extra and self.has_feed_forward and getattr(self.mixer, "folds_next_norm", False)
                and getattr(self.norm2, "folds_into_products", False)
                and getattr(self.feed_forward, "takes_scaled_rows", False)):
            extra["next_norm"] = self.norm2  # the norm between the two rides along with their products
        mixed = self.mixer.forward(x, batch, view, writes, **extra)
        if not self.has_feed_forward:
            return residual, mixed  # (the next norm adds it)
        x = normalise(self.norm2, residual, mixed, self.dtype)
        extra = {"residual": residual} if getattr(self.feed_forward, "adds_to_residual", False) else {}
        return residual, self.feed_forward.forward(x, **extra)


def normalise(norm, residual: torch.Tensor, pending, dtype: torch.dtype, rows=None):
    """Run ``norm`` on the residual stream plus what is pending.  Only a norm that
    says so (``takes_row_sumsq``) is shown the fused forms of a branch; for any
    other an already added branch becomes ``None``."""
    if not getattr(norm, "takes_row_sumsq", False) and isinstance(pending, (RowSumsq, Added)):
        pending = None
    if isinstance(pending, WeightedPair):
        pending = pending.combined()
    if rows is not None:
        return norm.forward(residual, pending, dtype, rows=rows)
    return norm.forward(residual, pending, dtype)


register_part("block", "pre_norm", PreNormBlock)


class BranchNormBlock(PreNormBlock):
    """``h += norm1(mixer(h)); h += norm2(feed_forward(h))``: no norm in front of a sublayer, one on its output.
    The stream is float32; each add (one kernel with the norm) also leaves the stream rounded to the activation
    type, which the next sublayer's products read (in a float32 engine they read the stream itself).  A layer
    without feed-forward has no second norm; a checkpoint that holds one all the same is accepted.  The norms are
    of a kind with ``add_normed`` (``rms_norm_one_plus``)."""

    reads_stream = True

    def __init__(self, spec: LayerSpec) -> None:
        super().__init__(spec)
        self.has_feed_forward = spec.feed_forward.kind != "none"
        for norm in (self.norm1, self.norm2):
            if not hasattr(norm, "add_normed"):
                raise ValueError("this arrangement takes norms that can add a normed branch (rms_norm_one_plus)")

    def _parts(self):
        parts = [("norm1", self.norm1), ("mixer", self.mixer)]
        if self.has_feed_forward:
            parts += [("norm2", self.norm2), ("feed_forward", self.feed_forward)]
        return parts

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out = super().expected_tensors(prefix)
        if not self.has_feed_forward:
            for name, spec in self.norm2.expected_tensors(f"{prefix}{self.spec.name_of('norm2')}.").items():
                out[name] = replace(spec, optional=True)
        return out

    def forward(self, residual: torch.Tensor, pending, batch, view, writes: bool = True):
        if isinstance(pending, StreamRows) and pending.rows is not None:
            x = pending.rows
        elif pending is None or isinstance(pending, Added):
            x = residual if self.dtype == torch.float32 else residual.to(self.dtype)
        else:
            raise ValueError("a branch that is still to be added cannot be handed to this arrangement")
        mixed = self.mixer.forward(x, batch, view, writes)
        x = self.norm1.add_normed(residual, mixed, self.dtype, want_rows=self.dtype != torch.float32)
        if self.has_feed_forward:
            fed = self.feed_forward.forward(residual if x is None else x)
            x = self.norm2.add_normed(residual, fed, self.dtype, want_rows=self.dtype != torch.float32)
        return residual, StreamRows(x)


register_part("block", "branch_norm", BranchNormBlock)


@dataclass
class NormedRows:
    """Stands where a pending branch would: the stream is whole, and these are its rows under the two norms of the
    block that comes next (a block whose last kernel makes them hands them on; ``second`` is ``None`` where that
    block has no feed-forward)."""

    first: torch.Tensor
    second: Optional[torch.Tensor]
    owner: Any  # the block they were made for


class ParallelDepthBlock:
    """A layer whose two branches read the same stream, and whose successor reads an average over the depth:

        X_new = x + mult * (mixer(norm1(x)) + feed_forward(norm2(x)))
        x     = sum_j average[j] * X_j        j = 0 .. depth + 1

    with X_0 the embedding's rows and X_(i+1) what layer i left (``X_new``), all float32.  The model keeps the
    ``X_j`` of a step (``keeps_history``) and hands them to every call.  ``average`` is the checkpoint tensor
    ``<layer>dwa`` with ``depth + 2`` numbers; ``mult`` and ``depth`` are the layer's options.  One kernel adds the
    branches, stores X_new, averages and makes the two norms of the block that follows (``link_next``); the first
    block of a model makes its own norms.  A layer without feed-forward has no second norm; a checkpoint that holds
    one all the same is accepted."""

    keeps_history = True

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.mult = float(spec.option("mult", 1.0))
        self.depth = int(spec.option("depth", 0))
        self.average_name = str(spec.option("average_name", "dwa"))
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)
        self.has_feed_forward = spec.feed_forward.kind != "none"
        self.norm2 = build_part("norm", spec.norm2)
        self.next_block: Any = None
        for norm in (self.norm1, self.norm2):
            if not hasattr(norm, "gain"):
                raise ValueError("this arrangement takes norms with one gain (rms_norm_scalar)")

    def link_next(self, block: Any) -> None:
        """The block that runs after this one (``None``: the last); its norms ride in this block's last kernel."""
        self.next_block = block if isinstance(block, ParallelDepthBlock) else None

    def _parts(self):
        parts = [("norm1", self.norm1), ("mixer", self.mixer)]
        if self.has_feed_forward:
            parts += [("norm2", self.norm2), ("feed_forward", self.feed_forward)]
        return parts

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out: dict[str, TensorSpec] = {}
        for role, part in self._parts():
            out.update(part.expected_tensors(f"{prefix}{self.spec.name_of(role)}."))
        if not self.has_feed_forward:
            for name, spec in self.norm2.expected_tensors(f"{prefix}{self.spec.name_of('norm2')}.").items():
                out[name] = replace(spec, optional=True)
        out[prefix + self.average_name] = TensorSpec((self.depth + 2,), init="norm", keeps_float32=True)
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        self.dtype = dtype
        for role, part in self._parts():
            part.bind(tensors, f"{prefix}{self.spec.name_of(role)}.", dtype, device)
        self.average = tensors[prefix + self.average_name].float().contiguous()

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._parts())

    def warm_up(self, rows: int) -> None:
        for _, part in self._parts():
            warm = getattr(part, "warm_up", None)
            if warm is not None:
                warm(rows)

    def gains(self) -> tuple:
        return (self.norm1.gain, self.norm2.gain) if self.has_feed_forward else (self.norm1.gain,)

    def forward(self, residual: torch.Tensor, pending, batch, view, writes: bool = True, history=None):
        if history is None:
            raise ValueError("a layer that averages over the depth needs the model to keep what every layer left")
        if isinstance(pending, NormedRows) and pending.owner is self:
            first, second = pending.first, pending.second
        else:
            if pending is not None and not isinstance(pending, (Added, NormedRows)):
                raise ValueError("a branch that is still to be added cannot be handed to this arrangement")
            _, normed = ops.depth_stream(residual, gains=self.gains(), out_dtype=self.dtype, eps=self.norm1.eps,
                                         want_stream=False)
            first, second = normed[0], normed[1] if len(normed) > 1 else None
        mixed = self.mixer.forward(first, batch, view, writes)
        fed = self.feed_forward.forward(second) if self.has_feed_forward else None
        follower = self.next_block
        stream, normed = ops.depth_stream(
            residual, mixed, fed, mult=self.mult, history=history, newest=self.depth + 1, weights=self.average,
            gains=follower.gains() if follower is not None else (), out_dtype=self.dtype,
            eps=follower.norm1.eps if follower is not None else self.norm1.eps)
        if follower is None:
            return stream, None
        return stream, NormedRows(normed[0], normed[1] if len(normed) > 1 else None, follower)


register_part("block", "parallel_depth_average", ParallelDepthBlock)


class SandwichNormBlock(PreNormBlock):
    """``h += s1 * norm1_out(mixer(norm1(h)))``, then ``h += s2 * norm2_out(feed_forward(norm2(h)))``: norms on both
    sides of a sublayer, and a learned scale per channel (``s1``, ``s2``: the checkpoint tensors ``<layer>ls1`` and
    ``<layer>ls2``, or whatever the spec's ``names`` call ``scale1`` and ``scale2``) on what joins the stream.  The
    scale is folded into the output norm's weight once, in float32.  One kernel norms a sublayer's output, adds it
    and makes the norm that the next sublayer reads (the next layer's first norm too, where that layer is of this
    kind), so the stream is read and written once per sublayer.  The output norms are of a kind with ``add_normed``
    (``rms_norm_groups`` with one group).  A layer without feed-forward has neither second norm nor ``s2``."""

    def __init__(self, spec: LayerSpec) -> None:
        super().__init__(spec)
        if spec.norm1_out is None or (self.has_feed_forward and spec.norm2_out is None):
            raise ValueError("this arrangement needs a norm for every sublayer's output (norm1_out, norm2_out)")
        self.norm1_out = build_part("norm", spec.norm1_out)
        self.norm2_out = build_part("norm", spec.norm2_out) if self.has_feed_forward else None
        self.layer_scale = bool(spec.option("layer_scale", True))
        for norm in (self.norm1_out, self.norm2_out):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ValueError("this arrangement takes output norms that can add a normed branch")
        self.next_block: Any = None

    def link_next(self, block: Any) -> None:
        """The block that runs after this one (``None``: the last); its first norm rides in this block's last kernel."""
        self.next_block = block if isinstance(block, SandwichNormBlock) else None

    def _parts(self):
        parts = [("norm1", self.norm1), ("mixer", self.mixer), ("norm1_out", self.norm1_out)]
        if self.has_feed_forward:
            parts += [("norm2", self.norm2), ("feed_forward", self.feed_forward), ("norm2_out", self.norm2_out)]
        return parts

    def _scales(self):
        if not self.layer_scale:
            return ()
        return ("scale1", "scale2") if self.has_feed_forward else ("scale1",)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out = super().expected_tensors(prefix)
        width = self.norm1.size
        for role in self._scales():
            out[prefix + self.spec.name_of(role)] = TensorSpec((width,), init="norm", keeps_float32=True)
        if not self.has_feed_forward:
            extra = dict(build_part("norm", self.spec.norm2_out).expected_tensors(f"{prefix}{self.spec.name_of('norm2_out')}.")
                         if self.spec.norm2_out is not None else {})
            if self.layer_scale:
                extra[prefix + self.spec.name_of("scale2")] = TensorSpec((width,), init="norm", keeps_float32=True)
            for name, spec in extra.items():
                out[name] = replace(spec, optional=True)
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        # the scale per channel and the output norm's weight multiply one after the other: their float32 product, once
        self.out_weight1 = self.norm1_out.weight_f32
        self.out_weight2 = self.norm2_out.weight_f32 if self.has_feed_forward else None
        if self.layer_scale:
            self.out_weight1 = (self.out_weight1 * tensors[prefix + self.spec.name_of("scale1")].float()).contiguous()
            if self.has_feed_forward:
                self.out_weight2 = (self.out_weight2 * tensors[prefix + self.spec.name_of("scale2")].float()).contiguous()

    def forward(self, residual: torch.Tensor, pending, batch, view, writes: bool = True):
        if isinstance(pending, NormedRows) and pending.owner is self:
            x = pending.first
        else:
            x = normalise(self.norm1, residual, pending, self.dtype)
        mixed = self.mixer.forward(x, batch, view, writes)
        follower = self.next_block
        after = follower.norm1.weight_f32 if follower is not None else None
        if self.has_feed_forward:
            _, x = self.norm1_out.add_normed(residual, mixed, self.dtype, weight=self.out_weight1,
                                             then=self.norm2.weight_f32)
            fed = self.feed_forward.forward(x)
            last = self.norm2_out.add_normed(residual, fed, self.dtype, weight=self.out_weight2, then=after)
        else:
            last = self.norm1_out.add_normed(residual, mixed, self.dtype, weight=self.out_weight1, then=after)
        if follower is None:
            return residual, None
        return residual, NormedRows(last[1], None, follower)


register_part("block", "sandwich_norm", SandwichNormBlock)
