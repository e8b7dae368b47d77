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
        # decode steps that are started before the tokens of the step before have arrived (see step())
        self._launch_decode = getattr(runner, "launch_decode", None)
        self._can_launch_decode = getattr(runner, "can_launch_decode", None)
        self.async_decode = bool(getattr(config, "async_decode", False)) and self._launch_decode is not None \
            and self._can_launch_decode is not None
        self._in_flight: tuple[BatchPlan, Any] | None = None  # (plan, its pending tokens)
        self._resolving = False

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
        if self._in_flight is not None and not self._resolving:
            self._take_in_flight()  # what it has generated so far is kept
            if request.is_terminal:
                return
        request.state = RequestState.CANCELLED
        request.finish_reason = "cancelled"
        self._finalize(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.active or self._in_flight is not None)

    def run_until_done(self, max_iterations: int | None = None) -> None:
        iterations = 0
        while self.has_work():
            self.step()
            iterations += 1
            if max_iterations is not None and iterations >= max_iterations:
                raise RuntimeError(f"scheduler did not drain in {max_iterations} iterations")

    def step(self) -> bool:
        """One iteration: admit, plan, run the plan, take the tokens.  Returns
        whether anything progressed.

        With ``async_decode`` a plan in which every request decodes one token is
        only started; its tokens are taken by the next call, after that call has
        started the step that follows (whose rows take their tokens on the device).
        The GPU then never waits for the host between two decode steps.  What the
        host cannot know in time is an end-of-sequence token: such a request runs
        one step more than needed, and that step's token is dropped."""
        if self._in_flight is not None:
            return self._step_behind_in_flight()
        progressed = self._admit_waiting()
        with trace_range("scheduler.build_batch_plan"):
            plan = self._build_batch_plan()
        if not plan.items:
            return progressed
        if self._may_launch(plan):
            try:
                with trace_range("scheduler.launch_decode"):
                    pending = self._launch_decode(plan, [-1] * len(plan.items),
                                                  [item.request.generated_count for item in plan.items])
            except Exception as exc:
                self._plan_failed(plan, exc)
                return True
            self._in_flight = (plan, pending)
            return True
        try:
            with trace_range("scheduler.execute_batch"):
                outputs = self.runner.execute_batch(plan)
        except Exception as exc:
            self._plan_failed(plan, exc)
            return True
        self._take_outputs(plan, outputs)
        return True

    def _plan_failed(self, plan: BatchPlan, exc: Exception) -> None:
        if bool(getattr(exc, "is_capacity_error", False)):
            if not self._preempt_for_capacity(plan):
                for item in plan.items:
                    if not item.request.is_terminal:
                        self._fail(item.request,
                                   f"KV capacity cannot fit one runnable sequence: {exc}", rejected=True)
            return
        for item in plan.items:
            if not item.request.is_terminal:
                self._fail(item.request, f"packed forward failed: {exc}")

    def _take_outputs(self, plan: BatchPlan, outputs: dict[str, int]) -> None:
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

    # -- decode steps whose tokens are taken one call later ------------------------------
    def _may_launch(self, plan: BatchPlan) -> bool:
        return (self.async_decode and all(item.is_decode and item.sample for item in plan.items)
                and self._can_launch_decode(len(plan.items)))

    def _take_in_flight(self) -> None:
        """Wait for the tokens of the step in flight and hand them to their requests."""
        plan, pending = self._in_flight
        self._in_flight = None
        self._resolving = True
        try:
            self._take_outputs(plan, pending.tokens())
        finally:
            self._resolving = False

    def _follow_up(self, plan: BatchPlan) -> tuple[BatchPlan, list[int], list[int]] | None:
        """The step after the one in flight, if it can be planned without that step's tokens: the same
        requests, less those that reach their token limit with the token in flight; each row takes its
        token from the place of its request in the step in flight."""
        if self.waiting and len(self.active) < self.config.max_running:
            return None  # a request wants in: let the step in flight end, then admit
        in_flight = {id(item.request) for item in plan.items}
        if any(id(request) not in in_flight for request in self.active if not request.is_terminal):
            return None  # someone still has a prompt to run: the next step is a mixed one
        items, feed, indices = [], [], []
        for place, item in enumerate(plan.items):
            request = item.request
            if request.is_terminal or request.generated_count + 1 >= request.config.max_output_tokens:
                continue
            items.append(BatchItem(request=request, token_ids=(0,), start_pos=request.tokens_fed, sample=True,
                                   is_decode=True))
            feed.append(place)
            indices.append(request.generated_count + 1)
        if not items or not self._can_launch_decode(len(items)):
            return None
        return BatchPlan(tuple(items)), feed, indices

    def _step_behind_in_flight(self) -> bool:
        plan, _ = self._in_flight
        follow = self._follow_up(plan) if self.async_decode else None
        launched = None
        failure: Exception | None = None
        if follow is not None:
            try:
                with trace_range("scheduler.launch_decode"):
                    launched = self._launch_decode(*follow)
            except Exception as exc:  # nothing was started; the tokens in flight are taken first
                failure = exc
        self._take_in_flight()
        if launched is not None:
            self._in_flight = (follow[0], launched)
        elif failure is not None and not bool(getattr(failure, "is_capacity_error", False)):
            self._plan_failed(follow[0], failure)
        # (a shortage of pages shows again in the next call, which plans with the tokens in hand and preempts)
        return True

    # -- internals -----------------------------------------------------------------
    def _room_beside_admitted(self, request: Request) -> bool:
        """Whether the pool holds what is known of ``request`` beside what is known
        of the admitted requests (the part of it that they have not taken yet)."""
        free_tokens = getattr(self.runner, "free_tokens", None)
        if free_tokens is None:
            return True
        allocated_tokens = getattr(self.runner, "allocated_tokens", lambda _r: 0)
        owed = 0
        for admitted in self.active:
            if not admitted.is_terminal:
                known = len(admitted.prompt_token_ids) + admitted.generated_count + 1
                owed += max(0, known - allocated_tokens(admitted))
        return free_tokens() - owed >= len(request.prompt_token_ids) + request.generated_count + 1

    def _admit_waiting(self) -> bool:
        progressed = False
        while self.waiting and len(self.active) < self.config.max_running:
            candidate = self.waiting[0]
            if candidate.preemption_count and self.active and not self._room_beside_admitted(candidate):
                # wait for room instead of thrashing; keeps its place at the head.  Room beside what the admitted
                # requests still have to take: the pages it has just given back are free, and taking them
                # again at once would starve the same requests again, for ever
                break
            if self.config.admit_within_pool and self.active and not self._room_beside_admitted(candidate):
                break  # admitted now it would push another request out, or be pushed out, and be computed twice
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
            prompt, generated = request.prompt_token_ids, request.generated_token_ids
            known = len(prompt) + len(generated)
            remaining = known - request.tokens_fed
            limit = 1 if candidate.phase == "decode" else self.config.prefill_chunk
            query_length = min(remaining, limit, budget)
            start = request.tokens_fed
            end = start + query_length
            # the portion's tokens, without joining the two lists (a decode step would copy the whole context)
            if start >= len(prompt):
                token_ids = tuple(generated[start - len(prompt): end - len(prompt)])
            elif end <= len(prompt):
                token_ids = tuple(prompt[start:end])
            else:
                token_ids = tuple(prompt[start:]) + tuple(generated[: end - len(prompt)])
            items.append(BatchItem(
                request=request,
                token_ids=token_ids,
                start_pos=start,
                sample=end == known,
                is_decode=query_length == 1 and start >= len(prompt),
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
