"""Request lifecycle and the iteration-level scheduler.

The policy is the reference's packed scheduler (src/cloud_engine/scheduler.py):
one state machine ``waiting -> prefill -> decoding -> completed | cancelled |
failed`` (:29-46); FIFO admission up to ``max_running`` (:438-457); each
iteration builds one plan under a shared token budget, decodes first, prompts
cut into portions of at most ``prefill_chunk`` tokens (:459-518); a sampled
token becomes the next iteration's one-token input (:581-607); EOS or
``max_output_tokens`` finishes a request (:593-605).  It is synchronous: the
caller drives :meth:`Scheduler.step`; streams, time-outs and the asyncio loop of
the reference belong to its server and are not here.

When pages run out (:527-553): the step raised a capacity error before changing
anything; the live request with the largest ``preemption_priority`` (most
resident tokens first) gives back all its pages and slot, keeps its generated
tokens, and goes to the *front* of the waiting queue with ``tokens_fed = 0``; it
is recomputed (prompt and generated tokens fed as prompt portions, sampling only
at the tail) once the pool has room for it again or nothing else is running.
The reference re-admits it only when nothing else runs and blocks the queue
behind it meanwhile (:443-446); here the queue is blocked too (a preempted
request keeps its seniority), but room in the pool suffices.  If a single live
request cannot get its pages, it fails with ``rejected`` set.
"""

from __future__ import annotations

import inspect
import time
from collections import deque
from collections.abc import Callable, Sequence
from dataclasses import dataclass, field
from enum import Enum
from typing import Any

from ..profiling import trace_range


class RequestState(Enum):
    WAITING = "waiting"
    PREFILL = "prefill"
    DECODING = "decoding"
    COMPLETED = "completed"
    CANCELLED = "cancelled"
    FAILED = "failed"


TERMINAL_STATES = frozenset({RequestState.COMPLETED, RequestState.CANCELLED, RequestState.FAILED})


class RejectionReason(Enum):
    QUEUE_FULL = "queue_full"
    KV_CAPACITY = "capacity_exhausted"
    CONTEXT_OVERFLOW = "context_length_exceeded"


class RejectedError(RuntimeError):
    def __init__(self, reason: RejectionReason, detail: str = "") -> None:
        super().__init__(detail or reason.value)
        self.reason = reason


@dataclass
class GenerationConfig:
    """``temperature == 0`` is greedy (all the reference samples with,
    src/cloud_engine/scheduler.py:63-71); ``temperature > 0`` draws from
    softmax(logits / temperature) with a generator keyed by ``seed`` and the
    token's index, so a request's draws do not depend on its batch.
    ``eos_token_id is None`` ignores EOS."""

    max_output_tokens: int
    temperature: float = 0.0
    eos_token_id: int | None = None
    seed: int | None = None

    def __post_init__(self) -> None:
        if self.max_output_tokens < 1:
            raise ValueError("max_output_tokens must be positive")
        if not self.temperature >= 0:
            raise ValueError("temperature must be zero (greedy) or positive")


@dataclass
class Request:
    request_id: str
    prompt_token_ids: list[int]
    config: GenerationConfig
    arrival_ns: int
    serial: int = 0
    label: str = ""
    state: RequestState = RequestState.WAITING
    generated_token_ids: list[int] = field(default_factory=list)
    tokens_fed: int = 0
    first_token_ns: int | None = None
    last_token_ns: int | None = None
    finish_ns: int | None = None
    finish_reason: str = ""
    error_detail: str = ""
    rejected: bool = False
    preemption_count: int = 0
    recomputed_tokens: int = 0
    recompute_until: int = 0
    on_token: Callable[["Request", int], None] | None = None

    @property
    def is_terminal(self) -> bool:
        return self.state in TERMINAL_STATES

    @property
    def generated_count(self) -> int:
        return len(self.generated_token_ids)


@dataclass(frozen=True)
class BatchItem:
    """One sequence's token slice in a shared iteration."""

    request: Request
    token_ids: tuple[int, ...]
    start_pos: int
    sample: bool
    is_decode: bool

    @property
    def query_length(self) -> int:
        return len(self.token_ids)

    @property
    def end_pos(self) -> int:
        return self.start_pos + self.query_length


@dataclass(frozen=True)
class BatchPlan:
    items: tuple[BatchItem, ...]

    @property
    def token_count(self) -> int:
        return sum(item.query_length for item in self.items)

    @property
    def request_ids(self) -> tuple[str, ...]:
        return tuple(item.request.request_id for item in self.items)


@dataclass(frozen=True)
class SchedulingCandidate:
    request_id: str
    phase: str
    remaining_tokens: int
    prompt_tokens: int
    generated_tokens: int
    arrival_ns: int


@dataclass(frozen=True)
class PreemptionCandidate:
    request_id: str
    allocated_tokens: int
    tokens_fed: int
    generated_tokens: int
    arrival_ns: int


def decode_first_priority(candidate: SchedulingCandidate) -> tuple[Any, ...]:
    """Decode before prefill; the stable sort keeps admission order inside each."""
    return (candidate.phase != "decode",)


def largest_sequence_preemption(candidate: PreemptionCandidate) -> tuple[Any, ...]:
    """Reclaim the most resident work first."""
    return (candidate.allocated_tokens, candidate.tokens_fed, candidate.arrival_ns)


class Scheduler:
    def __init__(
        self,
        config: Any,
        runner: Any,
        metrics: Any,
        clock: Callable[[], int] = time.monotonic_ns,
        scheduling_priority: Callable[[SchedulingCandidate], tuple[Any, ...]] = decode_first_priority,
        preemption_priority: Callable[[PreemptionCandidate], tuple[Any, ...]] = largest_sequence_preemption,
    ) -> None:
        self.config = config
        self.runner = runner
        self.metrics = metrics
        self.clock = clock
        self.scheduling_priority = scheduling_priority
        self.preemption_priority = preemption_priority
        self.waiting: deque[Request] = deque()
        self.active: list[Request] = []
        self.finished: deque[Request] = deque(maxlen=4096)
        self._counter = 0
        self._release_takes_flag = "preempted" in inspect.signature(runner.release).parameters
        self._publish_prefix = getattr(runner, "publish_prefix", None)

    # -- public ------------------------------------------------------------------
    def submit(self, prompt_token_ids: Sequence[int], gen_config: GenerationConfig, label: str = "",
               on_token: Callable[[Request, int], None] | None = None) -> Request:
        if len(prompt_token_ids) == 0:
            raise RejectedError(RejectionReason.CONTEXT_OVERFLOW, "empty prompt")
        if len(prompt_token_ids) + gen_config.max_output_tokens > self.config.max_model_len:
            raise RejectedError(RejectionReason.CONTEXT_OVERFLOW)
        if len(self.waiting) >= self.config.max_queue_size:
            raise RejectedError(RejectionReason.QUEUE_FULL)
        self._counter += 1
        request = Request(
            request_id=f"req-{self._counter:08d}",
            prompt_token_ids=[int(t) for t in prompt_token_ids],
            config=gen_config,
            arrival_ns=self.clock(),
            serial=self._counter,
            label=label,
            on_token=on_token,
        )
        self.waiting.append(request)
        return request

    def cancel(self, request: Request) -> None:
        """Idempotent; the request's pages go back at once."""
        if request.is_terminal:
            return
        request.state = RequestState.CANCELLED
        request.finish_reason = "cancelled"
        self._finalize(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.active)

    def run_until_done(self, max_iterations: int | None = None) -> None:
        iterations = 0
        while self.has_work():
            self.step()
            iterations += 1
            if max_iterations is not None and iterations >= max_iterations:
                raise RuntimeError(f"scheduler did not drain in {max_iterations} iterations")

    def step(self) -> bool:
        """One iteration: admit, plan, run the plan, take the tokens.  Returns
        whether anything progressed."""
        progressed = self._admit_waiting()
        with trace_range("scheduler.build_batch_plan"):
            plan = self._build_batch_plan()
        if not plan.items:
            return progressed
        try:
            with trace_range("scheduler.execute_batch"):
                outputs = self.runner.execute_batch(plan)
        except Exception as exc:
            if bool(getattr(exc, "is_capacity_error", False)):
                if not self._preempt_for_capacity(plan):
                    for item in plan.items:
                        if not item.request.is_terminal:
                            self._fail(item.request,
                                       f"KV capacity cannot fit one runnable sequence: {exc}", rejected=True)
                return True
            for item in plan.items:
                if not item.request.is_terminal:
                    self._fail(item.request, f"packed forward failed: {exc}")
            return True

        stamp = self.clock()
        self.metrics.record_input_tokens(plan.token_count)
        for item in plan.items:
            request = item.request
            if request.is_terminal:
                continue
            recomputed = max(0, min(item.end_pos, request.recompute_until) - item.start_pos)
            if recomputed:
                request.recomputed_tokens += recomputed
                self.metrics.record_recomputed_tokens(recomputed)
            if item.sample:
                token_id = outputs.get(request.request_id)
                if token_id is None:
                    self._fail(request, "packed runner omitted sampled token")
                    continue
                self._after_token(request, int(token_id), stamp)
            else:
                request.state = RequestState.PREFILL
        self.metrics.record_iteration(len(plan.items))
        return True

    # -- internals -----------------------------------------------------------------
    def _room_for(self, request: Request) -> bool:
        free_tokens = getattr(self.runner, "free_tokens", None)
        if free_tokens is None:
            return False
        known = len(request.prompt_token_ids) + request.generated_count
        return free_tokens() >= known + 1

    def _admit_waiting(self) -> bool:
        progressed = False
        while self.waiting and len(self.active) < self.config.max_running:
            candidate = self.waiting[0]
            if candidate.preemption_count and self.active and not self._room_for(candidate):
                break  # wait for room instead of thrashing; keeps its place at the head
            self.waiting.popleft()
            try:
                self.runner.admit(candidate)
            except Exception as exc:
                self._fail(candidate, f"admission refused: {exc}",
                           rejected=bool(getattr(exc, "is_capacity_error", False)))
                continue
            candidate.state = RequestState.PREFILL
            self.active.append(candidate)
            progressed = True
        return progressed

    def _build_batch_plan(self) -> BatchPlan:
        budget = self.config.token_budget
        candidates: list[tuple[SchedulingCandidate, Request]] = []
        for request in self.active:
            if request.is_terminal:
                continue
            known = len(request.prompt_token_ids) + request.generated_count
            remaining = known - request.tokens_fed
            if remaining <= 0:
                continue
            phase = "decode" if request.state is RequestState.DECODING and remaining == 1 else "prefill"
            candidates.append((
                SchedulingCandidate(request.request_id, phase, remaining, len(request.prompt_token_ids),
                                    request.generated_count, request.arrival_ns),
                request,
            ))
        items: list[BatchItem] = []
        for candidate, request in sorted(candidates, key=lambda pair: self.scheduling_priority(pair[0])):
            if budget <= 0:
                break
            known_ids = request.prompt_token_ids + request.generated_token_ids
            remaining = len(known_ids) - request.tokens_fed
            limit = 1 if candidate.phase == "decode" else self.config.prefill_chunk
            query_length = min(remaining, limit, budget)
            start = request.tokens_fed
            end = start + query_length
            items.append(BatchItem(
                request=request,
                token_ids=tuple(known_ids[start:end]),
                start_pos=start,
                sample=end == len(known_ids),
                is_decode=query_length == 1 and start >= len(request.prompt_token_ids),
            ))
            budget -= query_length
        return BatchPlan(tuple(items))

    def _preempt_for_capacity(self, plan: BatchPlan) -> bool:
        candidates = [request for request in self.active if not request.is_terminal]
        if len(candidates) <= 1:
            return False
        allocated_tokens = getattr(self.runner, "allocated_tokens", lambda _r: 0)
        victim = max(
            candidates,
            key=lambda request: self.preemption_priority(PreemptionCandidate(
                request.request_id, allocated_tokens(request), request.tokens_fed,
                request.generated_count, request.arrival_ns)),
        )
        self.active.remove(victim)
        self._release(victim, preempted=True)
        victim.recompute_until = victim.tokens_fed
        victim.tokens_fed = 0
        victim.preemption_count += 1
        victim.state = RequestState.WAITING
        self.waiting.appendleft(victim)
        self.metrics.inc_preempted()
        return True

    def _release(self, request: Request, preempted: bool = False) -> None:
        if self._release_takes_flag:
            self.runner.release(request, preempted=preempted)
        else:
            self.runner.release(request)

    def _after_token(self, request: Request, token_id: int, now: int) -> None:
        finished_prompt = request.state is RequestState.PREFILL
        request.generated_token_ids.append(token_id)
        if request.first_token_ns is None:
            request.first_token_ns = now
            self.metrics.record_ttft_ms((now - request.arrival_ns) / 1e6)
        else:
            self.metrics.record_itl_ms((now - (request.last_token_ns or now)) / 1e6)
        request.last_token_ns = now
        self.metrics.record_output_token(1)
        eos_hit = request.config.eos_token_id is not None and token_id == request.config.eos_token_id
        limit_hit = request.generated_count >= request.config.max_output_tokens
        if eos_hit:
            request.finish_reason = "eos_token_reached"
        elif limit_hit:
            request.finish_reason = "max_output_tokens_reached"
        if request.on_token is not None and not eos_hit:
            request.on_token(request, token_id)
        if eos_hit or limit_hit:
            request.state = RequestState.COMPLETED
            self._finalize(request)
        else:
            request.state = RequestState.DECODING
            if finished_prompt and self._publish_prefix is not None:
                # the prompt's full pages are final from here on: requests that arrive while this one
                # still decodes can already share them
                self._publish_prefix(request)

    def _fail(self, request: Request, detail: str, rejected: bool = False) -> None:
        if request.is_terminal:
            return
        request.rejected = rejected
        request.state = RequestState.FAILED
        request.error_detail = detail
        request.finish_reason = "failed"
        self._finalize(request)

    def _finalize(self, request: Request) -> None:
        """The one terminal funnel: leave the queues, give the cache back, count."""
        if request in self.active:
            self.active.remove(request)
        if request in self.waiting:
            self.waiting.remove(request)
        try:
            self._release(request)
        except Exception as exc:  # release must never break teardown
            request.error_detail = f"release error: {exc}"
        request.finish_ns = self.clock()
        self.finished.append(request)
        if request.state is RequestState.COMPLETED:
            self.metrics.record_e2e_ms((request.finish_ns - request.arrival_ns) / 1e6)
            self.metrics.inc_completed()
        elif request.state is RequestState.CANCELLED:
            self.metrics.inc_cancelled()
        elif request.rejected:
            self.metrics.inc_rejected()
        else:
            self.metrics.inc_failed()
