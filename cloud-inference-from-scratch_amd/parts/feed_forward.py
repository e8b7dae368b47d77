"""Gated feed-forward (SwiGLU): ``down(act(gate(x)) * up(x))`` without biases.

Reference: ``Qwen2MLP`` (src/cloud_engine/model.py:86-100).  Gate and up are
one fused product here, the activation and the multiply one kernel.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..weights.tensors import TensorSpec
from .base import Part, register_part
from .linear import linear


class GatedMLP(Part):
    graph_safe = True
    adds_to_residual = True
    takes_scaled_rows = True  # its first product applies the scale of rows that come without it
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu") -> None:
        if activation != "silu":
            raise ValueError(f"gated feed-forward runs silu only, got {activation!r}")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {
            prefix + "gate_proj.weight": TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + "up_proj.weight": TensorSpec((self.intermediate_size, self.hidden_size)),
            prefix + "down_proj.weight": TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.w_gate_up = torch.cat(
            [tensors[prefix + "gate_proj.weight"], tensors[prefix + "up_proj.weight"]], dim=0
        ).contiguous()
        self.w_down = tensors[prefix + "down_proj.weight"].contiguous()

    def warm_up(self, rows: int) -> None:
        self.forward(torch.zeros((rows, self.hidden_size), dtype=self.w_down.dtype, device=self.w_down.device))

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        return linear(linear(x, self.w_gate_up, epilogue="silu"), self.w_down, into=residual)


register_part("feed_forward", "gated_mlp", GatedMLP)
