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
"""

from __future__ import annotations

import torch

from .base import Part, register_part

_TABLES: dict[tuple, tuple[torch.Tensor, torch.Tensor]] = {}


class RotaryHalf(Part):
    graph_safe = True
    rotates = True

    def __init__(self, head_dim: int, theta: float, max_position: int, rotary_dim: int | None = None) -> None:
        rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if head_dim <= 0 or rotary_dim <= 0 or rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError(f"rotary_dim must be even, positive and at most the head size {head_dim}, got {rotary_dim}")
        if not theta > 0 or max_position <= 0:
            raise ValueError("rotary theta and max_position must be positive")
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.max_position = max_position

    def tables(self, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
        """(cos, sin), each float32 ``[max_position, rotary_dim/2]`` (the two halves
        of the reference's table are equal, so one half is kept)."""
        key = (self.rotary_dim, self.theta, self.max_position, str(device))
        if key not in _TABLES:
            inv_freq = 1.0 / (
                self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim)
            )
            positions = torch.arange(self.max_position, dtype=torch.float32)
            angles = positions[:, None] * inv_freq[None, :]
            _TABLES[key] = (angles.cos().to(device).contiguous(), angles.sin().to(device).contiguous())
        return _TABLES[key]


class NoPosition(Part):
    graph_safe = True
    """Keys and queries enter the mixer as projected."""

    rotates = False

    def __init__(self, head_dim: int = 0, max_position: int = 1) -> None:
        self.head_dim = head_dim
        self.rotary_dim = 0
        self.max_position = max_position

    def tables(self, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
        key = ("none", max(self.head_dim, 2), str(device))
        if key not in _TABLES:
            zeros = torch.zeros((1, max(self.head_dim, 2) // 2), dtype=torch.float32, device=device)
            _TABLES[key] = (zeros, zeros)
        return _TABLES[key]


register_part("position", "rotary_half", RotaryHalf)
register_part("position", "none", NoPosition)
