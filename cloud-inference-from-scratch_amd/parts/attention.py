"""Grouped-query softmax attention over the paged cache.

Reference: ``Qwen2Attention.project`` (src/cloud_engine/model.py:103-137),
``apply_rope`` (src/cloud_engine/attention.py:75-85), the KV write before the
read (src/cloud_engine/cache.py:398-413) and the ragged attention of
``kernel.py:324-405``: query head ``h`` reads KV head ``h // group``, scores are
``q.k / sqrt(D)``, a token sees every cached key up to itself.  Here q, k and v
are one fused product, rotation and cache write are one kernel, and sizes, bias
switches, scale, position encoding and an optional window are parameters.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache.manager import PagedKV
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, build_part, register_part
from .linear import linear


class Attention(Part):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qkv_bias: bool, out_bias: bool, position: PartSpec, window: Optional[int] = None,
                 scale: Optional[float] = None) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} key heads")
        if head_dim % 8 or head_dim > 256:
            raise ValueError(f"head_dim must be a multiple of 8 up to 256 for the attention kernels, got {head_dim}")
        if window is not None and window < 1:
            raise ValueError("window must be positive")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qkv_bias = qkv_bias
        self.out_bias = out_bias
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = build_part("position", position)

    def cache_need(self) -> PagedKV:
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        q_out = self.num_heads * self.head_dim
        kv_out = self.num_kv_heads * self.head_dim
        out = {
            prefix + "q_proj.weight": TensorSpec((q_out, self.hidden_size)),
            prefix + "k_proj.weight": TensorSpec((kv_out, self.hidden_size)),
            prefix + "v_proj.weight": TensorSpec((kv_out, self.hidden_size)),
            prefix + "o_proj.weight": TensorSpec((self.hidden_size, q_out)),
        }
        if self.qkv_bias:
            out[prefix + "q_proj.bias"] = TensorSpec((q_out,))
            out[prefix + "k_proj.bias"] = TensorSpec((kv_out,))
            out[prefix + "v_proj.bias"] = TensorSpec((kv_out,))
        if self.out_bias:
            out[prefix + "o_proj.bias"] = TensorSpec((self.hidden_size,))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        names = ("q_proj", "k_proj", "v_proj")
        self.w_qkv = torch.cat([tensors[f"{prefix}{n}.weight"] for n in names], dim=0).contiguous()
        self.b_qkv = (
            torch.cat([tensors[f"{prefix}{n}.bias"] for n in names], dim=0).contiguous()
            if self.qkv_bias else None
        )
        self.w_o = tensors[prefix + "o_proj.weight"].contiguous()
        self.b_o = tensors[prefix + "o_proj.bias"].contiguous() if self.out_bias else None
        self.cos, self.sin = self.position.tables(device)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if batch.max_context > self.position.max_position and self.position.rotates:
            raise ValueError(
                f"position {batch.max_context - 1} is beyond the rotary table of {self.position.max_position}"
            )
        qkv = linear(x, self.w_qkv, self.b_qkv)
        ops.rope_kv_write(qkv, self.cos, self.sin, batch.positions, batch.seq_of_token, batch.seq_slot,
                          view.block_table, view.k_pool, view.v_pool, self.num_heads, self.num_kv_heads,
                          self.head_dim, rotate=self.position.rotates, write_kv=writes)
        context = attend(qkv, batch, view, self.num_heads, self.num_kv_heads, self.head_dim,
                         self.window, self.scale)
        return linear(context, self.w_o, self.b_o)


def attend(qkv: torch.Tensor, batch, view, num_heads: int, num_kv_heads: int, head_dim: int,
           window: Optional[int], scale: float) -> torch.Tensor:
    """Pick the attention kernel for this step's rows."""
    return ops.paged_attention_generic(
        qkv, qkv.stride(0), view.k_pool, view.v_pool, view.block_table, batch.positions,
        batch.seq_of_token, batch.seq_slot, batch.tokens, num_heads, num_kv_heads, head_dim, window, scale)


register_part("mixer", "attention", Attention)
