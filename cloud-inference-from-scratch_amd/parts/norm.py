"""RMSNorm, fused with the residual add that precedes it.

Formula of the reference's ``rms_norm`` (src/cloud_engine/attention.py:52-57):
``x * rsqrt(mean(x^2) + eps) * weight`` with float32 statistics.  The reference
rounds the normalised value to the model dtype before the weight multiply; here
the multiply is float32 too and the result is rounded once.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, register_part
from .linear import Added, RowSumsq, ScaledRows, SummedBranch, WeightedPair


class RMSNorm(Part):
    graph_safe = True
    takes_row_sumsq = True
    # between a product that adds into the residual and a product that reads the norm's output, the norm can
    # ride along: the first writes residual * weight, the second applies the rows' 1 / rms to its sums
    folds_into_products = True
    def __init__(self, size: int, eps: float) -> None:
        if size <= 0 or not eps > 0:
            raise ValueError(f"RMSNorm needs a positive size and eps, got {size}, {eps}")
        if size > ops.MAX_NORM_WIDTH:
            raise ValueError(f"the norm kernels take rows of up to {ops.MAX_NORM_WIDTH} numbers, not {size}")
        self.size = size
        self.eps = eps
        self.weight: Optional[torch.Tensor] = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + "weight": TensorSpec((self.size,), init="norm", keeps_float32=True)}

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.weight = tensors[prefix + "weight"].contiguous()
        self.weight_f32 = self.weight.float().contiguous()

    def forward(self, residual: torch.Tensor, branch, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``branch`` is a tensor still to be added into ``residual``, ``None``, an
        ``Added`` (already added) or a ``RowSumsq`` (already added; the rows' sums
        of squares are known, so the norm needs no reduction)."""
        if isinstance(branch, Added):
            branch = None
        if isinstance(branch, RowSumsq):
            if branch.scaled is not None and branch.norm is self and rows is None and out_dtype == torch.bfloat16:
                return ScaledRows(branch.scaled, branch.sumsq, self.eps, residual, self)
            if rows is None and out_dtype == torch.bfloat16:
                return ops.rmsnorm_from_sumsq(residual, branch.sumsq, self.weight, self.eps)
            branch = None
        return ops.add_rmsnorm(residual, branch, self.weight, self.eps, out_dtype, rows=rows)


class ScalarRMSNorm(Part):
    """RMS norm with one gain for all coordinates: ``x * rsqrt(mean(x^2) + eps) * g``.  The checkpoint holds ``g``
    as a tensor without dimensions whose name is the norm's own (the prefix it is bound under, less the dot).
    Statistics and scaling are float32.  ``gain`` is what a kernel that makes this norm beside other work
    (``ops.depth_stream``) is given; ``forward`` serves everyone else through the vector norm's kernel."""

    graph_safe = True

    def __init__(self, size: int, eps: float) -> None:
        if size <= 0 or not eps > 0:
            raise ValueError(f"a norm needs a positive size and eps, got {size}, {eps}")
        if size > ops.MAX_NORM_WIDTH:
            raise ValueError(f"the norm kernels take rows of up to {ops.MAX_NORM_WIDTH} numbers, not {size}")
        self.size = size
        self.eps = eps
        self.gain = 1.0

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix.rstrip("."): TensorSpec((), init="norm", keeps_float32=True)}

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.gain = float(tensors[prefix.rstrip(".")].float().item())
        self.weight_f32 = torch.full((self.size,), self.gain, dtype=torch.float32, device=device)

    def forward(self, residual: torch.Tensor, branch, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(branch, (Added, RowSumsq)):
            branch = None
        return ops.add_rmsnorm(residual, branch, self.weight_f32, self.eps, out_dtype, rows=rows)


class OnePlusRMSNorm(RMSNorm):
    """RMS norm whose checkpoint weight lies around zero: ``x * rsqrt(mean(x^2) + eps) * (1 + w)``.  The sum
    ``1 + w`` is made once, in float32, when the weight is bound, and the tensor is named like the norm itself
    (no ``.weight``).  ``add_normed`` is the form a layer uses that norms its branches' outputs:
    ``residual += norm(branch)``."""

    folds_into_products = False  # (the products' norm epilogues multiply by a weight in the activation type)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix.rstrip("."): TensorSpec((self.size,), init="normal", keeps_float32=True)}

    def bind(self, tensors, prefix, dtype, device) -> None:
        Part.bind(self, tensors, prefix, dtype, device)
        self.weight = (1.0 + tensors[prefix.rstrip(".")].float()).contiguous()
        self.weight_f32 = self.weight

    def add_normed(self, residual: torch.Tensor, branch, out_dtype: torch.dtype, want_rows: bool = True):
        """``residual += norm(branch)`` in float32; returns the new stream in ``out_dtype`` (if wanted).
        ``branch`` is a tensor or a ``SummedBranch``."""
        main, parts = (branch.main, branch.parts) if isinstance(branch, SummedBranch) else (branch, None)
        if isinstance(branch, SummedBranch) and (branch.weights is not None or branch.main_gate is not None):
            raise ValueError("this norm sums a branch's rows as they are: weights and gates are not its to apply")
        return ops.branch_norm_add(residual, main, self.weight, self.eps, out_dtype, parts=parts, want_rows=want_rows)


class GroupedRMSNorm(Part):
    """RMS norm whose statistics run over ``groups`` equal consecutive parts of the row: each part is divided by
    its own ``sqrt(mean(part^2) + eps)``, and the whole row is multiplied by the weight.  One group is the plain RMS
    norm.  The tensor is named like the norm itself (no ``.weight``).  The kernel that norms also adds whatever a
    branch still owes the stream: a tensor, a ``SummedBranch`` (rows still to be summed, with weights per row where it
    has them, and a gate on its main tensor), and ``plus`` (float32 rows that join the stream before the norm, such
    as the embedding's rows once more).  Sums, statistics and scaling are float32."""

    graph_safe = True
    takes_plus = True

    def __init__(self, size: int, eps: float, groups: int = 1) -> None:
        if size <= 0 or not eps > 0 or groups < 1 or size % groups:
            raise ValueError(f"a norm of {size} numbers in {groups} groups with eps {eps}: sizes positive, groups that divide")
        if size + groups > ops.MAX_NORM_WIDTH:
            raise ValueError(f"the norm kernels take rows of up to {ops.MAX_NORM_WIDTH} numbers, not {size}")
        self.size, self.eps, self.groups = size, float(eps), groups
        self.weight: Optional[torch.Tensor] = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix.rstrip("."): TensorSpec((self.size,), init="norm", keeps_float32=True)}

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.weight = tensors[prefix.rstrip(".")].float().contiguous()
        self.weight_f32 = self.weight

    def forward(self, residual: torch.Tensor, branch, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None, plus: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(branch, (Added, RowSumsq)):
            branch = None
        extra = {}
        if isinstance(branch, SummedBranch):
            extra = dict(parts=branch.parts, part_weight=branch.weights, branch_gate=branch.main_gate)
            branch = branch.main
        return ops.group_norm_add(residual, branch, self.weight, self.groups, self.eps, out_dtype, rows=rows,
                                  plus=plus, **extra)


def _add_normed(self, residual: torch.Tensor, branch, out_dtype: torch.dtype, want_rows: bool = False,
                weight: Optional[torch.Tensor] = None, then: Optional[torch.Tensor] = None):
    """``residual += norm(branch) * weight`` in float32 and in place, for a norm of one group.  ``branch``: a
    tensor, a ``SummedBranch`` (rows still to be summed, with their weights and the gate on its main tensor) or a
    ``WeightedPair``.  ``weight`` (float32 [H]) stands in for the norm's own where the caller has folded a scale per
    channel into it.  ``then`` (float32 [H]): the RMS norm of the new stream under that weight comes back too.
    Returns what ``ops.branch_norm_add`` returns."""
    if self.groups != 1:
        raise ValueError("a norm on a sublayer's output takes its statistics over the whole row")
    extra = {}
    if isinstance(branch, SummedBranch):
        extra = dict(parts=branch.parts, part_weight=branch.weights, branch_gate=branch.main_gate)
        branch = branch.main
    elif isinstance(branch, WeightedPair):
        extra = dict(branch2=branch.second, scales=branch.scales)
        branch = branch.first
    return ops.branch_norm_add(residual, branch, self.weight if weight is None else weight, self.eps, out_dtype,
                               want_rows=want_rows, next_weight=then, **extra)


GroupedRMSNorm.add_normed = _add_normed

register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "rms_norm_groups", GroupedRMSNorm)
register_part("norm", "rms_norm_one_plus", OnePlusRMSNorm)
register_part("norm", "rms_norm_scalar", ScalarRMSNorm)
