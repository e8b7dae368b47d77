"""``x @ W^T + b`` for a Linear's weight ``[out, in]``, and its fused forms.

float32: the hand-written true-float32 kernel, always.  bfloat16 with up to
``FUSED_ROWS`` rows (decode steps): the hand-written matrix-core kernel that
streams the weight once and takes over its neighbours' work: an RMSNorm in front
(``LazyNorm`` input), a SiLU-gate behind (``epilogue="silu"``) or the add into
the float32 residual stream (``into=residual``).  bfloat16 with more rows: the
library product, as the reference leaves its products to a library
(src/cloud_engine/model.py:89-137), with the small kernels around it.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Union

import torch

from ..kernels import ops

# Rows up to which the hand-written fused bf16 kernel replaces the library product.
FUSED_ROWS = 16
# An ``into=`` product with fewer than this many 16-column tiles and K of at least 2 * PART_K cuts K
# into parts of about PART_K for more workgroups (partial products, summed by the next norm kernel).
PART_BELOW_TILES = 512
PART_K = 2752
# Fold a pending RMSNorm into the product's operand.  Measured on MI355X it loses: every workgroup
# re-reads and re-normalises the same few rows, and those reads pile up on a few cache channels; a
# separate small norm kernel from the known sums of squares is faster.  Kept for experiments.
FOLD_NORM = False


@dataclass
class RowSumsq:
    """Stands where a branch output would: the branch was already added into the
    residual stream, and ``sumsq`` [rows, parts] holds partial sums of squares of
    the residual's rows (what an RMSNorm needs of them)."""

    sumsq: torch.Tensor


@dataclass
class PartialSum:
    """Stands where a branch output would: float32 partial products ``parts``
    [P, rows, hidden] whose sum is the branch (a product whose K was cut)."""

    parts: torch.Tensor


@dataclass
class LazyNorm:
    """An RMSNorm that has not run: the consumer either folds it into its product
    or calls :meth:`materialize`."""

    residual: torch.Tensor
    sumsq: torch.Tensor
    weight: torch.Tensor
    eps: float
    dtype: torch.dtype

    @property
    def shape(self) -> torch.Size:
        return self.residual.shape

    def materialize(self) -> torch.Tensor:
        if self.dtype == torch.bfloat16:
            return ops.rmsnorm_from_sumsq(self.residual, self.sumsq, self.weight, self.eps)
        return ops.add_rmsnorm(self.residual, None, self.weight, self.eps, self.dtype)


def _fusable(rows: int, weight: torch.Tensor, silu: bool) -> bool:
    n, k = weight.shape
    return (weight.dtype == torch.bfloat16 and 1 <= rows <= FUSED_ROWS and k % 8 == 0
            and n % (32 if silu else 16) == 0)


def linear(x: Union[torch.Tensor, LazyNorm], weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, epilogue: Optional[str] = None,
           into: Optional[torch.Tensor] = None) -> Union[torch.Tensor, RowSumsq, PartialSum]:
    """``x @ weight.T + bias``.

    ``epilogue="silu"``: weight stacks gate rows over up rows; returns
    ``silu(gate) * up``.  ``into=residual``: the caller wants the result added to
    the float32 residual stream; if the fused kernel runs it adds it in place and
    a :class:`RowSumsq` comes back (or a :class:`PartialSum` of partial products
    that the next norm kernel adds), otherwise the plain result comes back and
    the caller adds it (the next norm kernel does)."""
    rows = x.shape[0]
    silu = epilogue == "silu"
    if _fusable(rows, weight, silu):
        if isinstance(x, LazyNorm) and not FOLD_NORM:
            x = x.materialize()
        source = (dict(residual_in=x.residual, sumsq_in=x.sumsq, norm_weight=x.weight, eps=x.eps)
                  if isinstance(x, LazyNorm) else dict(a=x))
        if into is not None:
            n, k = weight.shape
            if n // 16 < PART_BELOW_TILES and k >= 2 * PART_K:
                return PartialSum(ops.gemm_fused(weight, ops.EPI_PARTIAL, bias=bias, k_parts=-(-k // PART_K), **source))
            return RowSumsq(ops.gemm_fused(weight, ops.EPI_RESID, bias=bias, residual_out=into, **source))
        kind = ops.EPI_SILU if silu else ops.EPI_F32 if out_dtype == torch.float32 else ops.EPI_BF16
        return ops.gemm_fused(weight, kind, bias=bias, **source)
    if isinstance(x, LazyNorm):
        x = x.materialize()
    if weight.dtype == torch.float32:
        out = ops.gemm_f32(x, weight, bias)
    else:
        wanted = out_dtype or torch.bfloat16
        k = x.shape[1]
        ours = k % 8 == 0 and x.stride(0) % 8 == 0
        if ours and wanted == torch.float32:
            out = ops.gemm_bf16(x, weight, bias, wanted)
        elif wanted == torch.float32:
            # a shape the kernel refuses: widen the operands, exact products, float32 sums
            out = x.float() @ weight.float().t()
            out = out if bias is None else out + bias.float()
        else:
            out = torch.nn.functional.linear(x, weight, bias)
    return ops.silu_mul(out) if silu else out
