"""Decode steps as captured HIP graphs.

A step in which every request brings one token is launch-bound: a few hundred
small kernels per step.  As the reference does with CUDA graphs
(src/cloud_engine/engine.py:316-437) the whole forward of such a step is
captured once per power-of-two bucket of batch sizes and replayed.  All that
changes between replays lives in one static int32 buffer on the device (token
ids, positions, slots, context lengths, the step's longest context); kernels
read lengths from there, grids are fixed per bucket.  Rows of the bucket that no
request fills run as padding on the cache's pad slot and pad page.  Nothing is
cleared with a memset inside the graph.
"""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass
from typing import Any

import torch

from .batch import StepBatch, to_device_staging


@dataclass
class StaticPlan:
    """What kernel planning may use during a captured step: only bounds known at
    capture time and device tensors."""

    tile_seq: torch.Tensor      # int32 [bucket] = 0..bucket-1 (one query tile per sequence)
    tile_q0: torch.Tensor       # int32 [bucket] = 0
    max_context: torch.Tensor   # int32 [1], the step's longest context, rewritten before each replay
    max_keys: int               # upper bound of any context (max_model_len)


class _Bucket:
    def __init__(self, size: int, device: torch.device, pad_slot: int, max_keys: int,
                 token_pool: torch.Tensor | None = None) -> None:
        self.size = size
        count = 11 * size + 2
        self.host = torch.zeros(count, dtype=torch.int32)  # the template; every replay stages a copy of it
        self.dev = torch.zeros(count, dtype=torch.int32, device=device)
        names = ["token_ids", "positions", "seq_of_token", "seq_slot", "seq_start", "seq_q_len"]
        self.offsets: dict[str, int] = {}
        offset = 0
        for name in names:
            self.offsets[name] = offset
            offset += size
        self.offsets["q_start_loc"] = offset
        offset += size + 1
        for name in ("logit_rows", "tile_seq", "tile_q0", "token_feed"):
            self.offsets[name] = offset
            offset += size
        self.offsets["max_context"] = offset
        assert offset + 1 == count
        arange = torch.arange(size + 1, dtype=torch.int32)
        o = self.offsets
        self.host[o["seq_of_token"]: o["seq_of_token"] + size] = arange[:size]
        self.host[o["seq_q_len"]: o["seq_q_len"] + size] = 1
        self.host[o["q_start_loc"]: o["q_start_loc"] + size + 1] = arange
        self.host[o["logit_rows"]: o["logit_rows"] + size] = arange[:size]
        self.host[o["tile_seq"]: o["tile_seq"] + size] = arange[:size]
        self.pad_slot = pad_slot
        self.fill([], [], [], 1)
        self.dev.copy_(self.host)

        def view(name: str, length: int = size) -> torch.Tensor:
            return self.dev[o[name]: o[name] + length]

        self.batch = StepBatch(
            tokens=size, sequences=size, token_ids=view("token_ids"), positions=view("positions"),
            seq_of_token=view("seq_of_token"), seq_slot=view("seq_slot"), seq_start=view("seq_start"),
            seq_q_len=view("seq_q_len"), q_start_loc=view("q_start_loc", size + 1), logit_rows=view("logit_rows"),
            host_slots=[pad_slot] * size, host_starts=[0] * size, host_q_lens=[1] * size,
            static_plan=StaticPlan(view("tile_seq"), view("tile_q0"), view("max_context", 1), max_keys),
            token_feed=view("token_feed") if token_pool is not None else None, token_pool=token_pool,
        )
        self.graph: Any = None
        self.logits: torch.Tensor | None = None

    def fill(self, tokens: Sequence[int], positions: Sequence[int], slots: Sequence[int], max_context: int,
             feed: Sequence[int] | None = None) -> None:
        """Real rows first, the rest padding: token 0 at position 0 of the pad slot.  ``feed[i] >= 0``:
        row i takes the token at that place of the token pool on the device instead of ``tokens[i]``."""
        o, size, n = self.offsets, self.size, len(tokens)
        pad = size - n
        host = self.host
        host[o["token_feed"]: o["token_feed"] + size] = torch.tensor(
            (list(feed) if feed is not None else [-1] * n) + [-1] * pad, dtype=torch.int32)
        host[o["token_ids"]: o["token_ids"] + size] = torch.tensor(list(tokens) + [0] * pad, dtype=torch.int32)
        host[o["positions"]: o["positions"] + size] = torch.tensor(list(positions) + [0] * pad, dtype=torch.int32)
        host[o["seq_start"]: o["seq_start"] + size] = host[o["positions"]: o["positions"] + size]
        host[o["seq_slot"]: o["seq_slot"] + size] = torch.tensor(list(slots) + [self.pad_slot] * pad,
                                                                 dtype=torch.int32)
        host[o["max_context"]] = max(1, max_context)


class DecodeGraphs:
    def __init__(self, runner: Any, largest: int | None = None) -> None:
        self.runner = runner
        self.largest = largest or 1 << (max(runner.config.max_running, 1) - 1).bit_length()
        self.buckets: dict[int, _Bucket] = {}
        # the tokens the last step sampled, on the device: a step may start from them before the host has them
        self.token_pool = torch.zeros(self.largest, dtype=torch.int32, device=runner.device)
        self.pool: Any = None
        self.captures = 0
        self.replays = 0

    def takes(self, sequences: int) -> bool:
        return 1 <= sequences <= self.largest

    @staticmethod
    def bucket_of(sequences: int) -> int:
        return 1 << (sequences - 1).bit_length()

    def _capture(self, size: int) -> _Bucket:
        runner = self.runner
        bucket = _Bucket(size, runner.device, runner.device_cache.pad_slot, runner.config.max_model_len,
                         self.token_pool)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # first run outside capture: libraries set themselves up
            runner.model.forward(bucket.batch, runner.device_cache)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        with torch.cuda.graph(graph, pool=self.pool):
            bucket.logits = runner.model.forward(bucket.batch, runner.device_cache)
        bucket.graph = graph
        self.buckets[size] = bucket
        self.captures += 1
        return bucket

    def capture_all(self) -> int:
        """Capture every bucket that is not captured yet (rows of padding only), so that no later step
        pays for a capture; returns how many were made."""
        made = 0
        size = 1
        while size <= self.largest:
            if size not in self.buckets:
                self._capture(size)
                made += 1
            size *= 2
        return made

    def run(self, entries: Sequence[Any], feed: Sequence[int] | None = None) -> torch.Tensor:
        """Replay the bucket's graph for single-token entries; logits [wanted, vocab].  ``feed[i] >= 0``:
        entry i's token is the one at that place of ``token_pool`` (its own ``tokens`` are ignored)."""
        runner = self.runner
        size = self.bucket_of(len(entries))
        bucket = self.buckets.get(size) or self._capture(size)
        cache = runner.cache
        positions = [e.start_pos for e in entries]
        bucket.fill([e.tokens[0] for e in entries], positions, [cache.slot(e.request_id) for e in entries],
                    max(positions) + 1, feed)
        bucket.dev.copy_(to_device_staging(bucket.host, runner.device), non_blocking=True)
        bucket.graph.replay()
        self.replays += 1
        rows = [index for index, e in enumerate(entries) for _ in e.want]
        if rows == list(range(len(entries))):
            return bucket.logits[: len(entries)]
        return bucket.logits[torch.tensor(rows, dtype=torch.long, device=runner.device)]
