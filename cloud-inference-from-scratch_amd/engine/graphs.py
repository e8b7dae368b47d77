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

import contextlib
import gc
from collections.abc import Iterator, Sequence
from dataclasses import dataclass
from typing import Any

import torch

from .batch import StepBatch, to_device_staging


@dataclass
class StaticPlan:
    """What kernel planning may use during a captured step: only bounds known at
    capture time and device tensors."""

    tile_seq: torch.Tensor | None  # int32 [bucket] = 0..bucket-1 (one query tile per sequence)
    tile_q0: torch.Tensor | None   # int32 [bucket] = 0
    max_context: torch.Tensor   # int32 [1], the step's longest context, rewritten before each replay
    max_keys: int               # upper bound of any context (max_model_len, or the bound a captured step was made for)
    decode_rows: int | None = None  # the step's first sequences that bring one token each; None: all of them


@contextlib.contextmanager
def _collector_off() -> Iterator[None]:
    """Around a capture.  A runner and its graphs refer to each other, so a runner that is gone waits for
    the cyclic collector with its captured graphs; a graph destroyed while another is being captured aborts
    the process.  What waits is collected now, and the collector stays off until the capture has ended."""
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if was_enabled:
            gc.enable()


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
        with _collector_off(), torch.cuda.graph(graph, pool=self.pool):
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

    def run(self, entries: Sequence[Any], feed: Sequence[int] | None = None, borrow: bool = False) -> torch.Tensor:
        """Replay the bucket's graph for single-token entries; logits [wanted, vocab].  ``feed[i] >= 0``:
        entry i's token is the one at that place of ``token_pool`` (its own ``tokens`` are ignored).
        The graph writes its logits into one buffer of its own, which the bucket's next replay overwrites:
        the caller gets a copy, unless it ``borrow``s the buffer (sampling that is queued on the same
        stream right behind the replay has read it before the next replay can start)."""
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
            view = bucket.logits[: len(entries)]
            return view if borrow else view.clone()
        # (the index goes over as an asynchronous copy: a tensor made on the device from a list would wait for the replay)
        index = to_device_staging(rows, runner.device).to(runner.device, non_blocking=True).long()
        return bucket.logits.index_select(0, index)


@dataclass
class _CapturedStep:
    """A captured step of single tokens beside prompt portions, and the buffer its replays rewrite."""

    decode_rows: int
    portions: tuple[int, ...]
    host: torch.Tensor
    dev: torch.Tensor
    offsets: dict[str, int]
    batch: StepBatch
    graph: Any = None
    logits: torch.Tensor | None = None
    # which rows of ``logits`` a step's entries want, as index tensors on the device, by the rows' numbers: made
    # once each (a tensor made on the device from a host list waits for the stream, that is for the replay)
    wanted_rows: dict = None


class MixedGraphs:
    """Steps that bring short prompt portions (beside decode tokens or alone) as captured graphs.

    Such a step is a few hundred launches too, and with few tokens the host cannot queue them as fast as the
    GPU runs them (8 decode rows and a 32-token portion of the 3B shape: 4.1 ms launch by launch, 3.6 ms
    replayed; with a 64-token portion 4.4 and 4.2 ms; with 256 tokens the GPU is the slower one either way).  A capture costs as
    much as ten such steps, so only shapes that come again are captured: a step's shape is (bucket of its
    single-token rows, the lengths of its portions); one that comes a second time (the portions of one
    long prompt beside the same decoding requests do) is captured, on rows of padding, and replayed from
    then on.  As in captured decode steps, the parts of the
    keys are sized on the device from the step's longest context.  The least recently used shapes beyond
    ``limit`` are dropped.  The reference captures decode steps only (src/cloud_engine/engine.py:316-437)."""

    MAX_PORTIONS = 4
    MAX_TOKENS = 128  # rows of a step (decode bucket and portions) up to which the host is the slower side

    def __init__(self, runner: Any, decode_graphs: "DecodeGraphs", limit: int) -> None:
        self.runner = runner
        self.decode_graphs = decode_graphs
        self.limit = limit
        self.steps: dict[tuple, _CapturedStep] = {}   # in order of last use
        self.seen: dict[tuple, int] = {}
        self.captures = 0
        self.replays = 0

    def shape_of(self, entries: Sequence[Any]) -> tuple | None:
        """The step's shape if a captured graph may run it, else None: at most MAX_PORTIONS portions, and
        logits wanted at no other place than a portion's last token."""
        single = [e for e in entries if len(e.tokens) == 1]
        portions = [e for e in entries if len(e.tokens) > 1]
        if not portions or len(portions) > self.MAX_PORTIONS or len(single) > self.decode_graphs.largest:
            return None
        bucket = DecodeGraphs.bucket_of(len(single)) if single else 0
        if bucket + sum(len(e.tokens) for e in portions) > self.MAX_TOKENS:
            return None
        for e in portions:
            if tuple(e.want) not in ((), (len(e.tokens) - 1,)):
                return None
        if any(len(e.want) > 1 for e in single):
            return None
        return bucket, tuple(len(e.tokens) for e in portions)

    def wants(self, entries: Sequence[Any]) -> tuple | None:
        """The shape if this step is to run from a graph now (captured already, or seen before)."""
        if self.limit < 1:
            return None
        shape = self.shape_of(entries)
        if shape is None:
            return None
        if shape in self.steps:
            return shape
        self.seen[shape] = self.seen.get(shape, 0) + 1
        if len(self.seen) > 4096:
            self.seen.clear()
        return shape if self.seen[shape] >= 2 else None

    def _layout(self, shape: tuple) -> _CapturedStep:
        decode_rows, portions = shape
        runner = self.runner
        bound = runner.config.max_model_len
        sequences = decode_rows + len(portions)
        tokens = decode_rows + sum(portions)
        offsets: dict[str, int] = {}
        offset = 0
        for name, length in (("token_ids", tokens), ("positions", tokens), ("seq_of_token", tokens),
                             ("seq_slot", sequences), ("seq_start", sequences), ("seq_q_len", sequences),
                             ("q_start_loc", sequences + 1), ("logit_rows", sequences), ("max_context", 1)):
            offsets[name] = offset
            offset += length
        host = torch.zeros(offset, dtype=torch.int32)
        q_lens = [1] * decode_rows + list(portions)
        starts = [0]
        for count in q_lens:
            starts.append(starts[-1] + count)
        o = offsets
        host[o["seq_of_token"]: o["seq_of_token"] + tokens] = torch.tensor(
            [index for index, count in enumerate(q_lens) for _ in range(count)], dtype=torch.int32)
        host[o["seq_q_len"]: o["seq_q_len"] + sequences] = torch.tensor(q_lens, dtype=torch.int32)
        host[o["q_start_loc"]: o["q_start_loc"] + sequences + 1] = torch.tensor(starts, dtype=torch.int32)
        # logits: every single-token row, and the last token of every portion
        host[o["logit_rows"]: o["logit_rows"] + sequences] = torch.tensor(
            [start + count - 1 for start, count in zip(starts, q_lens)], dtype=torch.int32)
        dev = torch.zeros(offset, dtype=torch.int32, device=runner.device)

        def view(name: str, length: int) -> torch.Tensor:
            return dev[o[name]: o[name] + length]

        pad = runner.device_cache.pad_slot
        batch = StepBatch(
            tokens=tokens, sequences=sequences, token_ids=view("token_ids", tokens), positions=view("positions", tokens),
            seq_of_token=view("seq_of_token", tokens), seq_slot=view("seq_slot", sequences),
            seq_start=view("seq_start", sequences), seq_q_len=view("seq_q_len", sequences),
            q_start_loc=view("q_start_loc", sequences + 1), logit_rows=view("logit_rows", sequences),
            host_slots=[pad] * sequences, host_starts=[0] * sequences, host_q_lens=q_lens,
            static_plan=StaticPlan(None, None, view("max_context", 1), bound, decode_rows=decode_rows),
        )
        return _CapturedStep(decode_rows, portions, host, dev, offsets, batch, wanted_rows={})

    def _fill(self, step: _CapturedStep, single: Sequence[Any], portions: Sequence[Any]) -> None:
        """Real single-token rows first, padding up to the bucket (token 0 at position 0 of the pad slot),
        then the portions."""
        cache = self.runner.cache
        pad = step.decode_rows - len(single)
        tokens = [e.tokens[0] for e in single] + [0] * pad
        positions = [e.start_pos for e in single] + [0] * pad
        slots = [cache.slot(e.request_id) for e in single] + [self.runner.device_cache.pad_slot] * pad
        starts = list(positions)
        for e in portions:
            tokens.extend(e.tokens)
            positions.extend(range(e.start_pos, e.start_pos + len(e.tokens)))
            slots.append(cache.slot(e.request_id))
            starts.append(e.start_pos)
        o, host = step.offsets, step.host
        host[o["token_ids"]: o["token_ids"] + len(tokens)] = torch.tensor(tokens, dtype=torch.int32)
        host[o["positions"]: o["positions"] + len(positions)] = torch.tensor(positions, dtype=torch.int32)
        host[o["seq_slot"]: o["seq_slot"] + len(slots)] = torch.tensor(slots, dtype=torch.int32)
        host[o["seq_start"]: o["seq_start"] + len(starts)] = torch.tensor(starts, dtype=torch.int32)
        host[o["max_context"]] = max(e.start_pos + len(e.tokens) for e in list(single) + list(portions))
        step.dev.copy_(to_device_staging(host, self.runner.device), non_blocking=True)

    def _fill_padding(self, step: _CapturedStep) -> None:
        """Every row padding: token 0 on the pad slot, the portions at positions 0, 1, ... of it (its block
        table names the pad page at every place)."""
        o, host = step.offsets, step.host
        positions = [0] * step.decode_rows + [p for count in step.portions for p in range(count)]
        sequences = step.decode_rows + len(step.portions)
        host[o["token_ids"]: o["token_ids"] + len(positions)] = 0
        host[o["positions"]: o["positions"] + len(positions)] = torch.tensor(positions, dtype=torch.int32)
        host[o["seq_slot"]: o["seq_slot"] + sequences] = self.runner.device_cache.pad_slot
        host[o["seq_start"]: o["seq_start"] + sequences] = 0
        host[o["max_context"]] = max(step.portions)
        step.dev.copy_(to_device_staging(host, self.runner.device), non_blocking=True)

    def _capture(self, step: _CapturedStep) -> None:
        """Capture on rows of padding, as the decode steps are: the run before the capture (libraries set
        themselves up, tile lists are made) and the capture itself touch the pad slot and the pad page only,
        so that a part which keeps a state per request (and would advance it at every run) sees each of the
        step's tokens once, at the replay."""
        runner = self.runner
        self._fill_padding(step)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            runner.model.forward(step.batch, runner.device_cache)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        if self.decode_graphs.pool is None:
            self.decode_graphs.pool = torch.cuda.graph_pool_handle()
        with _collector_off(), torch.cuda.graph(graph, pool=self.decode_graphs.pool):
            step.logits = runner.model.forward(step.batch, runner.device_cache)
        step.graph = graph
        self.captures += 1

    def run(self, shape: tuple, entries: Sequence[Any]) -> torch.Tensor:
        """Replay (after capturing, if need be) the graph of this shape; logits [wanted, vocab] in the order
        of the entries."""
        single = [e for e in entries if len(e.tokens) == 1]
        portions = [e for e in entries if len(e.tokens) > 1]
        step = self.steps.pop(shape, None)
        if step is None:
            step = self._layout(shape)
            self._capture(step)  # (a capture that fails leaves no half-made entry behind)
        self._fill(step, single, portions)
        self.steps[shape] = step  # last in the order of use
        while len(self.steps) > self.limit:
            del self.steps[next(iter(self.steps))]
        step.graph.replay()
        self.replays += 1
        row_of = {id(e): index for index, e in enumerate(single)}
        row_of.update({id(e): step.decode_rows + index for index, e in enumerate(portions)})
        rows = tuple(row_of[id(e)] for e in entries for _ in e.want)
        index = step.wanted_rows.get(rows)
        if index is None:
            if len(step.wanted_rows) > 64:
                step.wanted_rows.clear()
            index = step.wanted_rows[rows] = to_device_staging(list(rows), self.runner.device).to(
                self.runner.device, non_blocking=True).long()
        return step.logits.index_select(0, index)
