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


def to_device_staging(values: Any, device: torch.device | str) -> torch.Tensor:
    """int32 values (a list, or a CPU tensor) in host memory that an asynchronous copy to ``device`` may
    read later: a fresh page-locked tensor from torch's caching host allocator, which hands a block out
    again only after the copies that read it have run.  (A page-locked buffer of one's own that is
    rewritten step after step would be overwritten under a copy that is still queued behind earlier
    kernels, whenever the host runs ahead of the GPU.)"""
    pinned = torch.device(device).type == "cuda"
    if isinstance(values, torch.Tensor):
        staged = torch.empty(values.shape, dtype=torch.int32, pin_memory=pinned)
        staged.copy_(values)
        return staged
    return torch.tensor(values, dtype=torch.int32, pin_memory=pinned)


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
    # filled for a step that replays a captured graph: everything a kernel plan reads comes from the device
    static_plan: Any = None
    # a decode step that follows one whose tokens the host has not seen yet: row t takes token_pool[token_feed[t]]
    # where token_feed[t] >= 0 (both int32 on the device)
    token_feed: Any = None
    token_pool: Any = None
    _tiles: dict = field(default_factory=dict)

    @property
    def all_decode(self) -> bool:
        return all(n == 1 for n in self.host_q_lens)

    @property
    def max_q_len(self) -> int:
        return max(self.host_q_lens, default=0)

    def tiles(self, tokens_per_tile: int, decode: bool | None) -> tuple[torch.Tensor, torch.Tensor, int]:
        """Query tiles of at most ``tokens_per_tile`` consecutive tokens of one
        sequence, for the sequences that bring one token (``decode``), more (``decode=False``)
        or any number (``decode=None``):
        (sequence index of each tile, its first token within the sequence's
        portion, number of tiles), the two lists as int32 device tensors."""
        key = (tokens_per_tile, decode)
        if key not in self._tiles:
            seqs: list[int] = []
            firsts: list[int] = []
            for index, count in enumerate(self.host_q_lens):
                if decode is not None and (count == 1) != decode:
                    continue
                for first in range(0, count, tokens_per_tile):
                    seqs.append(index)
                    firsts.append(first)
            if seqs:
                both = to_device_staging(seqs + firsts, self.token_ids.device).to(self.token_ids.device, non_blocking=True)
                self._tiles[key] = (both[: len(seqs)], both[len(seqs):], len(seqs))
            else:
                self._tiles[key] = (self.seq_slot, self.seq_slot, 0)
        return self._tiles[key]

    @property
    def max_context(self) -> int:
        return max((s + n for s, n in zip(self.host_starts, self.host_q_lens)), default=0)


@dataclass
class PagedView:
    """One cache unit of paged keys and values, as a mixer sees it."""

    k_pool: torch.Tensor         # [pages, kv_heads, page_size, head_dim]
    v_pool: torch.Tensor | None  # [pages, kv_heads, value_width, page_size]  (transposed); None: keys only
    block_table: torch.Tensor    # int32 [max_running, width] of the unit's group
    page_size: int


@dataclass
class StateView:
    """One cache unit of fixed-size per-request state: row ``slot`` is the request's."""

    state: torch.Tensor          # [max_running, *shape]
    extra: Any = None
