"""Arrangement of a layer's parts.

``PreNormBlock``: the reference's decoder layer (src/cloud_engine/model.py:211-220)
``h += mixer(norm1(h)); h += feed_forward(norm2(h))``.  The residual stream is
float32; a branch's output is added inside the next norm kernel, so the block
returns the feed-forward output as ``pending`` instead of adding it.  A part
that can add its output into the residual itself (the fused decode products do)
returns a ``RowSumsq`` or an ``Added`` instead, and the next norm then runs its
cheaper form or rides along with the product behind it (``parts/linear.py``).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..config.specs import LayerSpec
from ..weights.tensors import TensorSpec
from .base import build_part, register_part
from .linear import Added, RawRows, RowSumsq


class PreNormBlock:
    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        self.norm2 = build_part("norm", spec.norm2)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)

    def _parts(self):
        return (("norm1", self.norm1), ("mixer", self.mixer), ("norm2", self.norm2),
                ("feed_forward", self.feed_forward))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        out: dict[str, TensorSpec] = {}
        for role, part in self._parts():
            out.update(part.expected_tensors(f"{prefix}{self.spec.name_of(role)}."))
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
                writes: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
        if ((pending is None or isinstance(pending, Added)) and getattr(self.mixer, "takes_raw_rows", False)
                and getattr(self.norm1, "folds_into_products", False) and RawRows.fits(residual, self.dtype)):
            # a few rows, the stream complete: the mixer's first product makes the norm itself (a kernel less)
            x = RawRows(residual, self.norm1, self.dtype)
        else:
            x = normalise(self.norm1, residual, pending, self.dtype)
        extra = {"residual": residual} if getattr(self.mixer, "adds_to_residual", False) else {}
        if (extra and getattr(self.mixer, "folds_next_norm", False) and getattr(self.norm2, "folds_into_products", False)
                and getattr(self.feed_forward, "takes_scaled_rows", False)):
            extra["next_norm"] = self.norm2  # the norm between the two rides along with their products
        mixed = self.mixer.forward(x, batch, view, writes, **extra)
        x = normalise(self.norm2, residual, mixed, self.dtype)
        extra = {"residual": residual} if getattr(self.feed_forward, "adds_to_residual", False) else {}
        return residual, self.feed_forward.forward(x, **extra)


def normalise(norm, residual: torch.Tensor, pending, dtype: torch.dtype, rows=None):
    """Run ``norm`` on the residual stream plus what is pending.  Only a norm that
    says so (``takes_row_sumsq``) is shown the fused forms of a branch; for any
    other an already added branch becomes ``None``."""
    if not getattr(norm, "takes_row_sumsq", False) and isinstance(pending, (RowSumsq, Added)):
        pending = None
    if rows is not None:
        return norm.forward(residual, pending, dtype, rows=rows)
    return norm.forward(residual, pending, dtype)


register_part("block", "pre_norm", PreNormBlock)
