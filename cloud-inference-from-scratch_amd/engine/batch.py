"""What one step hands to the model: the flat token axis and its metadata.

Plays the role of the reference's ``PackedContext``/``PackedBatch``
(src/cloud_engine/attention.py:35-49, src/cloud_engine/engine.py:60-67).  The
tokens of one sequence are contiguous on the flat axis, sequences in the order
of the step's entries.  Device tensors are int32 views into one staging buffer
that is uploaded with a single copy; the host lists serve kernel planning and
mixers that walk sequences on the host.  A slot mapping is not carried: kernels
derive a token's cache slot from the block table and its position.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import torch


@dataclass
class StepBatch:
    tokens: int
    sequences: int
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]   absolute position of each token
    seq_of_token: torch.Tensor   # int32 [T]   index of the token's sequence in this step
    seq_slot: torch.Tensor       # int32 [S]   the request's slot (row of block tables and states)
    seq_start: torch.Tensor      # int32 [S]   tokens cached before this step (context length)
    seq_q_len: torch.Tensor      # int32 [S]   tokens fed in this step
    q_start_loc: torch.Tensor    # int32 [S+1] offsets of the sequences on the flat axis
    logit_rows: torch.Tensor     # int32 [n]   flat rows whose logits are wanted
    host_slots: list[int] = field(default_factory=list)
    host_starts: list[int] = field(default_factory=list)
    host_q_lens: list[int] = field(default_factory=list)
    request_ids: tuple[str, ...] = ()

    @property
    def all_decode(self) -> bool:
        return all(n == 1 for n in self.host_q_lens)

    @property
    def max_q_len(self) -> int:
        return max(self.host_q_lens, default=0)

    @property
    def max_context(self) -> int:
        return max((s + n for s, n in zip(self.host_starts, self.host_q_lens)), default=0)


@dataclass
class PagedView:
    """One cache unit of paged keys and values, as a mixer sees it."""

    k_pool: torch.Tensor         # [pages, kv_heads, page_size, head_dim]
    v_pool: torch.Tensor
    block_table: torch.Tensor    # int32 [max_running, width] of the unit's group
    page_size: int


@dataclass
class StateView:
    """One cache unit of fixed-size per-request state: row ``slot`` is the request's."""

    state: torch.Tensor          # [max_running, *shape]
    extra: Any = None
