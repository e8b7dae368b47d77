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
from .linear import Added, RowSumsq, ScaledRows


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


register_part("norm", "rms_norm", RMSNorm)
