"""The step function: a batch of (request, its next tokens) in, logits out.

Counterpart of the reference's ``RaggedRunner`` (src/cloud_engine/engine.py:193-488):
``admit`` / ``release`` / ``allocated_tokens`` are what the scheduler calls;
:meth:`Runner.run` grows the cache all-or-nothing, packs the step's tokens on
one flat axis (prompt portions beside single decode tokens, cut anywhere), runs
the model once on exactly these tokens against the cache earlier steps left,
commits the lengths and returns float32 logits at the wanted places.  Unlike
the reference it returns logits at *any* wanted position and leaves sampling to
the caller, so trace replay and generation drive the same function.
"""

from __future__ import annotations

import itertools
from collections import deque
from collections.abc import Sequence
from dataclasses import dataclass, field
from typing import Any

import numpy as np
import torch

from ..cache.manager import CacheManager, PagedKV
from ..config.engine_config import EngineConfig
from ..kernels import ops
from ..profiling import trace_range
from ..sampling.sampler import Sampler
from .batch import StepBatch
from .device_cache import DeviceCache
from .graphs import DecodeGraphs, MixedGraphs


@dataclass(frozen=True)
class StepEntry:
    """One request's share of a step: its next ``tokens`` starting at
    ``start_pos`` (which must equal what the cache holds for it) and the places
    among these tokens whose logits are wanted."""

    request_id: str
    tokens: Sequence[int]
    start_pos: int
    want: Sequence[int] = field(default_factory=tuple)


@dataclass
class PendingTokens:
    """The tokens a launched decode step samples, on their way to the host."""

    request_ids: tuple[str, ...]
    host: torch.Tensor          # page-locked int32 [n]; valid once ``ready`` has passed
    ready: Any                  # torch.cuda.Event behind the copy

    def tokens(self) -> dict[str, int]:
        self.ready.synchronize()
        return dict(zip(self.request_ids, self.host.tolist()))


# What a running engine needs of the device memory beside weights and cache, set aside before the cache takes
# its share of what is free: the vendor library's workspace, the copies of a weight its timing runs stream
# through (gemm_library.hip keeps up to 640 MB of them while a shape's candidates are timed), and a full step's
# activations (per token and number of the model's width: the float32 stream, the 16-bit rows of the norms,
# projections and feed-forward, and partial sums, some 64 bytes) and float32 logits.
LIBRARY_TIMING_BYTES = 640 << 20
ACTIVATION_BYTES_PER_NUMBER = 64


def flat_needs(needs: Sequence[Any]) -> list[Any]:
    """The needs of a model's cache units, a unit of several needs spread out."""
    out: list[Any] = []
    for need in needs:
        out.extend(need) if isinstance(need, (tuple, list)) else out.append(need)
    return out


def reserve_bytes(config: EngineConfig, hidden_size: int, vocab_size: int) -> int:
    """Device memory kept out of the cache's reach (see above)."""
    reserve = ops.LIBRARY_WORKSPACE_BYTES
    if config.search_library_algorithms:
        reserve += LIBRARY_TIMING_BYTES
    reserve += config.token_budget * hidden_size * ACTIVATION_BYTES_PER_NUMBER
    reserve += 2 * config.max_running * vocab_size * 4
    return reserve


def tokens_from_bytes(config: EngineConfig, needs: Sequence[Any], element_bytes: int, free_bytes: int,
                      hidden_size: int, vocab_size: int) -> int:
    """The pool's size in tokens where none is given: ``kv_cache_bytes``, or ``kv_cache_fraction`` of the
    ``free_bytes`` that are left once :func:`reserve_bytes` is set aside; never more than every slot full and
    the prefix index can use, never less than one page."""
    per_token = sum(n.numbers_per_token * element_bytes for n in flat_needs(needs) if isinstance(n, PagedKV))
    page = config.page_size
    if per_token == 0:
        return page
    budget = config.kv_cache_bytes
    if budget is None:
        budget = int(max(0, free_bytes - reserve_bytes(config, hidden_size, vocab_size)) * config.kv_cache_fraction)
    tokens = budget // per_token
    useful = (config.max_running * -(-config.max_model_len // page) + config.prefix_cache_pages) * page
    return max(page, min(tokens, useful) // page * page)


class Runner:
    def __init__(self, model: Any, config: EngineConfig, device: str | torch.device = "cuda:0") -> None:
        if not torch.cuda.is_available():
            raise RuntimeError("the engine runs on the GPU only; no GPU is visible")
        self.model = model
        self.config = config
        self.device = torch.device(device)
        self.dtype = model.dtype
        needs = model.cache_needs()
        max_position = model.spec.max_position
        if config.max_model_len > max_position:
            raise ValueError(f"max_model_len {config.max_model_len} exceeds the model's {max_position} positions")
        kv_tokens = config.kv_tokens if config.kv_tokens is not None else self._tokens_from_bytes(needs)
        self.cache = CacheManager(
            needs, config.page_size, kv_tokens, config.max_running, config.max_model_len,
            prefill_chunk=config.prefill_chunk, prefix_cache_pages=config.prefix_cache_pages,
            element_bytes=torch.tensor([], dtype=self.dtype).element_size(),
        )
        self.device_cache = DeviceCache(self.cache, self.dtype, self.device)
        self.forward_invocations = 0
        self.max_forward_request_count = 0
        self.forward_plans: deque[tuple[tuple[str, int, int, int], ...]] = deque(maxlen=256)
        self.sampler = Sampler(config.seed)
        self.graphs = DecodeGraphs(self) if config.graph_decode and getattr(model, "graph_safe", False) else None
        self.mixed_graphs = (MixedGraphs(self, self.graphs, config.graph_mixed_steps)
                             if self.graphs is not None and config.graph_mixed_steps > 0 else None)
        self._staging = [None, None]
        self._staging_turn = 0
        # the row counts whose products time every algorithm of the vendor library: this engine's full steps
        self.search_rows = (frozenset({config.token_budget, min(config.prefill_chunk, config.token_budget)})
                            if config.search_library_algorithms else frozenset())

    def _tokens_from_bytes(self, needs: list[Any]) -> int:
        free = 0
        if self.config.kv_cache_bytes is None:
            free, _total = torch.cuda.mem_get_info(self.device)
        spec = self.model.spec
        return tokens_from_bytes(self.config, needs, torch.tensor([], dtype=self.dtype).element_size(), free,
                                 spec.hidden_size, spec.vocab_size)

    # -- what the scheduler calls ------------------------------------------------
    def admit(self, request: Any) -> None:
        request.cached = self.cache.admit(request.request_id, request.prompt)

    def release(self, request: Any, preempted: bool = False) -> None:
        self.cache.release(request.request_id, None if preempted else request.prompt)

    def warm_up(self) -> int:
        """Do now what the first steps would otherwise do on the clock: capture the decode graphs of
        all bucket sizes, and let the products of full prompt portions (one request's portion, and the
        sizes up to the token budget that time the library's candidates) set themselves up.  Returns
        the number of graphs captured."""
        with ops.library_search(self.search_rows):
            captured = self.graphs.capture_all() if self.graphs is not None else 0
            budget, chunk = self.config.token_budget, min(self.config.prefill_chunk, self.config.token_budget)
            rows = {chunk} | {n for n in range(512, budget + 1, 256)}
            warm = getattr(self.model, "warm_up", None)
            if warm is not None:
                warm(sorted(rows))
        return captured

    def publish_prefix(self, request: Any) -> None:
        """The request's prompt is in the cache: offer its full pages to the prefix index now, not only
        when it ends (the reference stores at release, src/cloud_engine/engine.py:224-226)."""
        self.cache.publish_prefix(request.request_id, request.prompt)

    def allocated_tokens(self, request: Any) -> int:
        return self.cache.allocated_tokens(request.request_id)

    @property
    def graph_captures(self) -> int:
        return self.graphs.captures if self.graphs is not None else 0

    @property
    def graph_replays(self) -> int:
        return self.graphs.replays if self.graphs is not None else 0

    @property
    def mixed_graph_captures(self) -> int:
        return self.mixed_graphs.captures if self.mixed_graphs is not None else 0

    @property
    def mixed_graph_replays(self) -> int:
        return self.mixed_graphs.replays if self.mixed_graphs is not None else 0

    def free_tokens(self) -> int:
        """Tokens the pool could take now (see :meth:`CacheManager.free_tokens`)."""
        return self.cache.free_tokens()

    def tokens_needed(self, request: Any, upto: int) -> int:
        """What the request would still take of :meth:`free_tokens` to hold ``upto`` tokens: whole pages, in
        the group that is shortest of them; a group that keeps a window only never asks for more than the
        window's pages; a cache without pages asks for nothing."""
        return self.cache.tokens_missing(request.request_id, upto)

    def execute_batch(self, plan: Any) -> dict[str, int]:
        """Run a scheduler's plan and sample where it asks to (the reference's
        ``execute_batch``, src/cloud_engine/engine.py:439-488)."""
        entries = [
            StepEntry(portion.request.request_id, portion.tokens, portion.start,
                      (portion.length - 1,) if portion.samples else ())
            for portion in plan.portions
        ]
        logits = self.run(entries, borrow_logits=True)  # (sampled from at once, below)
        for portion in plan.portions:
            portion.request.cached = portion.end
        sampling = [portion.request for portion in plan.portions if portion.samples]
        if not sampling:
            return {}
        with trace_range("ragged.sample"):
            tokens = self.sampler.sample(
                logits,
                [r.gen.temperature for r in sampling],
                [self.sampler.uniform(r.gen.seed, r.serial, len(r.output)) if r.gen.temperature > 0 else 0.0
                 for r in sampling],
            )
        return {r.request_id: token for r, token in zip(sampling, tokens)}

    # -- decode steps that do not wait for their tokens -----------------------------------
    def can_launch_decode(self, requests: int) -> bool:
        """Whether a step of that many single tokens can be started without waiting (a captured graph takes it)."""
        return self.graphs is not None and self.graphs.takes(requests)

    def launch_decode(self, plan: Any, feed: Sequence[int], token_indices: Sequence[int]) -> "PendingTokens":
        """Start a step in which every request brings one token and samples, and return at once.

        ``feed[i] >= 0``: portion i's token is the one the launch before this sampled at that place (it is
        still on the device; the portion's own token id is a placeholder).  ``token_indices[i]`` is the index of
        the token portion i is about to sample (what its random draw depends on).  The sampled tokens stay
        on the device for the next launch and travel to the host behind the step;
        :meth:`PendingTokens.tokens` waits for them."""
        assert self.graphs is not None and all(p.length == 1 and p.samples for p in plan.portions)
        entries = [StepEntry(p.request.request_id, p.tokens, p.start, (0,)) for p in plan.portions]
        logits = self.run(entries, feed=feed, borrow_logits=True)
        requests = [p.request for p in plan.portions]
        for p in plan.portions:
            p.request.cached = p.end
        with trace_range("ragged.sample"):
            pool = self.graphs.token_pool[: len(requests)]
            self.sampler.sample_on_device(
                logits, [r.gen.temperature for r in requests],
                [self.sampler.uniform(r.gen.seed, r.serial, index) if r.gen.temperature > 0 else 0.0
                 for r, index in zip(requests, token_indices)],
                out=pool)
            host = torch.empty(len(requests), dtype=torch.int32, pin_memory=True)
            host.copy_(pool, non_blocking=True)
            ready = torch.cuda.Event()
            ready.record()
        return PendingTokens(tuple(r.request_id for r in requests), host, ready)

    # -- packing -----------------------------------------------------------------
    def _stage(self, count: int) -> torch.Tensor:
        """The device buffer a step's metadata is copied into.  Two take turns: the copy of the next step
        is ordered on the stream behind the kernels that read the buffer two steps earlier."""
        turn = self._staging_turn
        self._staging_turn ^= 1
        dev = self._staging[turn]
        if dev is None or dev.numel() < count:
            dev = torch.empty(max(1024, 1 << (count - 1).bit_length()), dtype=torch.int32, device=self.device)
            self._staging[turn] = dev
        return dev

    def check(self, entries: Sequence[StepEntry]) -> None:
        """Refuse a step the kernels were not written for, before anything changes."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        vocab = self.model.spec.vocab_size
        seen: set[str] = set()
        for entry in entries:
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id} appears twice in one step")
            seen.add(entry.request_id)
            count = len(entry.tokens)
            if count == 0:
                raise ValueError(f"request {entry.request_id} brings no tokens")
            held = self.cache.length(entry.request_id)
            if entry.start_pos != held:
                raise ValueError(
                    f"request {entry.request_id} continues at {entry.start_pos} but the cache holds {held} tokens"
                )
            if not (0 <= min(entry.tokens) and max(entry.tokens) < vocab):  # (two passes at C speed; a prompt portion has thousands)
                token = next(t for t in entry.tokens if not 0 <= t < vocab)
                raise ValueError(f"token id {token} outside the vocabulary of {vocab}")
            for place in entry.want:
                if not 0 <= place < count:
                    raise ValueError(f"wanted place {place} outside the {count} tokens of {entry.request_id}")

    def pack(self, entries: Sequence[StepEntry]) -> StepBatch:
        """The step's metadata, laid out in one page-locked buffer and copied to the device once.  What has an
        entry per token (ids, positions, sequence of the token) is made by array operations, not token by token:
        a prompt portion of 2,048 tokens took 0.4 ms of lists here, before the step's first kernel could start."""
        count_of = [len(entry.tokens) for entry in entries]
        sequences = len(entries)
        total = sum(count_of)
        slots = [self.cache.slot(entry.request_id) for entry in entries]
        starts = [entry.start_pos for entry in entries]
        q_start_loc = [0]
        for count in count_of:
            q_start_loc.append(q_start_loc[-1] + count)
        logit_rows = [q_start_loc[index] + place for index, entry in enumerate(entries) for place in entry.want]
        sizes = [total, total, total, sequences, sequences, sequences, sequences + 1, len(logit_rows)]
        staged = torch.empty(sum(sizes), dtype=torch.int32, pin_memory=self.device.type == "cuda")
        host = staged.numpy()
        bounds = [0]
        for size in sizes:
            bounds.append(bounds[-1] + size)
        part = [host[bounds[i]: bounds[i + 1]] for i in range(len(sizes))]
        counts = np.asarray(count_of, dtype=np.int32)
        part[0][:] = np.fromiter(itertools.chain.from_iterable(entry.tokens for entry in entries), dtype=np.int32,
                                 count=total)
        part[2][:] = np.repeat(np.arange(sequences, dtype=np.int32), counts)
        # a token's position: its place on the flat axis, less its sequence's first place, plus the sequence's start
        shift = np.asarray(starts, dtype=np.int32) - np.asarray(q_start_loc[:-1], dtype=np.int32)
        part[1][:] = np.arange(total, dtype=np.int32) + np.repeat(shift, counts)
        part[3][:] = slots
        part[4][:] = starts
        part[5][:] = count_of
        part[6][:] = q_start_loc
        part[7][:] = logit_rows
        dev = self._stage(staged.numel())
        dev[: staged.numel()].copy_(staged, non_blocking=True)
        views = [dev[bounds[i]: bounds[i + 1]] for i in range(len(sizes))]
        return StepBatch(
            tokens=total, sequences=sequences, token_ids=views[0], positions=views[1],
            seq_of_token=views[2], seq_slot=views[3], seq_start=views[4], seq_q_len=views[5],
            q_start_loc=views[6], logit_rows=views[7], host_slots=slots, host_starts=starts,
            host_q_lens=count_of, request_ids=tuple(e.request_id for e in entries),
        )

    # -- the step ------------------------------------------------------------------
    def run(self, entries: Sequence[StepEntry], feed: Sequence[int] | None = None,
            borrow_logits: bool = False) -> torch.Tensor:
        """One step.  Returns float32 logits ``[sum(len(e.want)), vocab]`` on the
        device, in the order of the entries and of their ``want``; they are the
        caller's to keep.  Raises ``CacheCapacityFull`` before anything changes if
        pages run out.  ``feed`` (captured decode steps only): see
        :meth:`launch_decode`, which also borrows a captured step's own logits
        buffer instead of a copy (``borrow_logits``)."""
        self.check(entries)
        required = {e.request_id: e.start_pos + len(e.tokens) for e in entries}
        with trace_range("ragged.kv.ensure_capacity"):
            self.cache.ensure_capacity_batch(required)
            self.device_cache.sync()
        self.forward_invocations += 1
        self.max_forward_request_count = max(self.max_forward_request_count, len(entries))
        self.forward_plans.append(
            tuple((e.request_id, e.start_pos, len(e.tokens), len(e.want)) for e in entries)
        )
        decode = all(len(e.tokens) == 1 for e in entries)
        tokens = sum(len(e.tokens) for e in entries)
        with trace_range(f"ragged.forward.{'decode' if decode else 'mixed'}.requests_{len(entries)}.tokens_{tokens}"), \
                ops.library_search(self.search_rows):
            shape = None
            if not decode and feed is None and self.mixed_graphs is not None:
                shape = self.mixed_graphs.wants(entries)
            if decode and self.graphs is not None and self.graphs.takes(len(entries)):
                logits = self.graphs.run(entries, feed, borrow=borrow_logits)
            elif feed is not None:
                raise ValueError("tokens can be fed on the device to captured decode steps only")
            elif shape is not None:
                logits = self.mixed_graphs.run(shape, entries)
            else:
                logits = self.model.forward(self.pack(entries), self.device_cache)
        with trace_range("ragged.kv.commit"):
            self.cache.commit_lengths(required)
            self.device_cache.sync()
        return logits
