"""``x @ W^T + b`` for a Linear's weight ``[out, in]``.

float32: the hand-written true-float32 kernel, always.  bfloat16: for few rows
the hand-written matrix-core kernel that streams the weight once (decode steps
and the output head, which wants float32 logits); for many rows the library
product, as the reference leaves its products to a library
(src/cloud_engine/model.py:89-137).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops

# Rows up to which the hand-written bf16 kernel is used instead of the library.
SKINNY_ROWS = 0


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    if weight.dtype == torch.float32:
        return ops.gemm_f32(x, weight, bias)
    out_dtype = out_dtype or torch.bfloat16
    rows, k = x.shape
    ours = k % 8 == 0 and x.stride(0) % 8 == 0
    if ours and (out_dtype == torch.float32 or rows <= SKINNY_ROWS):
        return ops.gemm_bf16(x, weight, bias, out_dtype)
    if out_dtype == torch.float32:
        # a shape the kernel refuses: widen the operands, exact products, float32 sums
        out = x.float() @ weight.float().t()
        return out if bias is None else out + bias.float()
    return torch.nn.functional.linear(x, weight, bias)
