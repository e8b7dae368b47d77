"""Arrangement of a layer's parts.

``PreNormBlock``: the reference's decoder layer (src/cloud_engine/model.py:211-220)
``h += mixer(norm1(h)); h += feed_forward(norm2(h))``.  The residual stream is
float32; a branch's output is added inside the next norm kernel, so the block
returns the feed-forward output as ``pending`` instead of adding it.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..config.specs import LayerSpec
from ..weights.tensors import TensorSpec
from .base import build_part, register_part


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

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], batch, view,
                writes: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
        x = self.norm1.forward(residual, pending, self.dtype)
        mixed = self.mixer.forward(x, batch, view, writes)
        x = self.norm2.forward(residual, mixed, self.dtype)
        return residual, self.feed_forward.forward(x)


register_part("block", "pre_norm", PreNormBlock)
