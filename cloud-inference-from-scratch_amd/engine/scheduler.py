"""The iteration-level scheduler: which requests run in the next step, with how
many tokens each, and what happens when the pool cannot hold them.

The policy is that of the reference's packed scheduler
(src/cloud_engine/scheduler.py): requests are admitted in the order they came,
up to ``max_running`` (:438-457); every iteration shares one token budget, the
requests that decode go first and prompts are cut into portions of at most
``prefill_chunk`` tokens (:459-518); only a portion that reaches the request's
last known token samples (:513); the sampled token is the next iteration's
one-token portion, and an end-of-sequence token or ``max_output_tokens`` ends
the request (:581-607).  The loop is the caller's: :meth:`Scheduler.step` is one
iteration.  Streams, time-outs and the asyncio task of the reference belong to
its server and are not here.

**When pages run out** the step function has refused the plan before it changed
anything.  The live request that ranks highest under ``victim_order`` (most
resident tokens, as in the reference, :197-199, :527-553) gives back its pages
and its slot, keeps the tokens it has produced, and returns to the *front* of
the waiting queue; it comes back when the pool has room for everything known of
it beside what the admitted requests still have to take, or when nothing else
runs, and then rebuilds its cache from prompt + output as prompt portions.  (The
reference puts it at the back and lets it in only once nothing runs, :443-446.)
While it waits nobody behind it is admitted: it keeps its seniority.  A lone
request that cannot get its pages fails as ``rejected``.

**Decode steps in flight** (``async_decode``): a plan of single sampled tokens is
only started; the next call first starts the step that follows it, whose rows
take their tokens from the device, and then collects the tokens of the step
before.  Requests leave the follow-up in time when their token limit is in
sight; an end-of-sequence token is seen one step late and costs one dropped row.
"""

from __future__ import annotations

import inspect
import time
from collections import deque
from collections.abc import Callable, Sequence
from typing import Any

from ..profiling import trace_range
from .plan import Portion, Standing, StepPlan, decodes_before_prompts, most_resident_gives_way
from .request import GenerationConfig, Refusal, RejectedError, Request, RequestState

__all__ = ["GenerationConfig", "Portion", "Refusal", "RejectedError", "Request", "RequestState", "Scheduler",
           "Standing", "StepPlan", "decodes_before_prompts", "most_resident_gives_way"]

Order = Callable[[Standing], tuple[Any, ...]]


def _is_shortage(error: BaseException) -> bool:
    """The step function marks "no pages left" with an attribute, not a type, so that a
    scheduler needs nothing of the cache's modules (src/cloud_engine/scheduler.py:384)."""
    return bool(getattr(error, "is_capacity_error", False))


class _InFlight:
    """A started decode step: its plan, and the handle its tokens arrive through."""

    __slots__ = ("plan", "handle")

    def __init__(self, plan: StepPlan, handle: Any) -> None:
        self.plan = plan
        self.handle = handle


class Scheduler:
    def __init__(self, config: Any, runner: Any, metrics: Any, clock: Callable[[], int] = time.monotonic_ns,
                 plan_order: Order = decodes_before_prompts, victim_order: Order = most_resident_gives_way) -> None:
        self.config = config
        self.runner = runner
        self.metrics = metrics
        self.clock = clock
        self.plan_order = plan_order
        self.victim_order = victim_order
        self.waiting: deque[Request] = deque()
        self.active: list[Request] = []
        self.finished: deque[Request] = deque(maxlen=4096)
        self._submitted = 0
        # what the runner offers beyond admit / release / execute_batch
        self._release_knows_preemption = "preempted" in inspect.signature(runner.release).parameters
        self._resident = getattr(runner, "allocated_tokens", None)
        self._free = getattr(runner, "free_tokens", None)
        self._needed = getattr(runner, "tokens_needed", None)
        self._publish = getattr(runner, "publish_prefix", None)
        self._launch = getattr(runner, "launch_decode", None)
        self._launchable = getattr(runner, "can_launch_decode", None)
        self.async_decode = (bool(getattr(config, "async_decode", False))
                             and self._launch is not None and self._launchable is not None)
        self._flying: _InFlight | None = None
        self._collecting = False
        # a step has just failed for want of pages and one request has given way: nobody is let in until
        # those that stayed have run a step (else the one that gave way comes straight back, the step fails
        # again, and so on for ever if the guard at admission errs on the side of room)
        self._gave_way = False

    # ---------------------------------------------------------------- callers
    def submit(self, prompt: Sequence[int], gen: GenerationConfig, label: str = "",
               on_token: Callable[[Request, int], None] | None = None) -> Request:
        """Queue a request, or refuse it (src/cloud_engine/scheduler.py:233-254): no
        prompt, prompt + output beyond ``max_model_len``, queue full."""
        limits = self.config
        if not len(prompt):
            raise RejectedError(Refusal.TOO_LONG, "empty prompt")
        if len(prompt) + gen.max_output_tokens > limits.max_model_len:
            raise RejectedError(Refusal.TOO_LONG)
        if len(self.waiting) >= limits.max_queue_size:
            raise RejectedError(Refusal.QUEUE_FULL)
        self._submitted += 1
        serial = self._submitted
        request = Request(request_id="req-%08d" % serial, serial=serial, prompt=tuple(int(t) for t in prompt),
                          gen=gen, arrived_ns=self.clock(), label=label, on_token=on_token)
        self.waiting.append(request)
        return request

    def cancel(self, request: Request) -> None:
        """End a request now; its pages go back at once.  A second call does nothing."""
        if request.is_final:
            return
        if self._flying is not None and not self._collecting:
            self._collect()  # the token under way is kept
            if request.is_final:
                return
        self._retire(request, RequestState.CANCELLED, "cancelled")

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self.active) or self._flying is not None

    def run_until_done(self, max_iterations: int | None = None) -> None:
        done = 0
        while self.has_work():
            self.step()
            done += 1
            if max_iterations is not None and done >= max_iterations:
                raise RuntimeError(f"scheduler did not drain in {max_iterations} iterations")

    def step(self) -> bool:
        """One iteration.  Returns whether anything moved."""
        if self._flying is not None:
            self._step_behind()
            return True
        moved = self._admit()
        with trace_range("scheduler.build_batch_plan"):
            plan = self._plan()
        if not plan:
            return moved
        if self.async_decode and plan.all_decode and self._launchable(len(plan.portions)):
            self._start(plan)
        else:
            self._run(plan)
        return True

    # ---------------------------------------------------------------- admission
    def _fits_beside_admitted(self, request: Request) -> bool:
        """Whether the pool has room for all that is known of ``request`` once the admitted
        requests have taken what is known of them (plus the token each is about to sample)."""
        if self._free is None:
            return True
        needed = self._needed
        if needed is None:
            # a runner that does not say what a request costs it: whole pages of ``page_size`` per token
            # (one more token can cost a page), less what the request holds
            page = max(1, int(getattr(self.config, "page_size", 1)))
            resident = self._resident if self._resident is not None else (lambda _request: 0)
            needed = lambda r, upto: max(0, -(-upto // page) * page - resident(r))
        spoken_for = sum(needed(other, other.known + 1) for other in self.active if not other.is_final)
        return self._free() - spoken_for >= needed(request, request.known + 1)

    def _admit(self) -> bool:
        moved = False
        while self.waiting and len(self.active) < self.config.max_running and not (self._gave_way and self.active):
            head = self.waiting[0]
            # A preempted request that came back the moment its own pages were free would take them from
            # the same requests again, for ever.  A newcomer that does not fit would push someone out or
            # be pushed out, and be computed twice.  Both wait at the head; alone, anything may try.
            guarded = head.preemptions > 0 or self.config.admit_within_pool
            if guarded and self.active and not self._fits_beside_admitted(head):
                break
            self.waiting.popleft()
            try:
                self.runner.admit(head)
            except Exception as error:
                self._retire(head, RequestState.FAILED, "failed", error=f"admission refused: {error}",
                             rejected=_is_shortage(error))
                continue
            head.state = RequestState.PREFILL
            self.active.append(head)
            moved = True
        return moved

    # ---------------------------------------------------------------- planning
    def _plan(self) -> StepPlan:
        runnable = [r for r in self.active if not r.is_final and r.pending > 0]
        standings = {id(r): Standing.of(r) for r in runnable}
        runnable.sort(key=lambda r: self.plan_order(standings[id(r)]))
        left = self.config.token_budget
        portions: list[Portion] = []
        for request in runnable:
            if left <= 0:
                break
            most = 1 if standings[id(request)].decoding else self.config.prefill_chunk
            take = min(request.pending, most, left)
            start = request.cached
            portions.append(Portion(request, start, request.tokens(start, start + take),
                                    samples=start + take == request.known))
            left -= take
        return StepPlan(tuple(portions))

    # ---------------------------------------------------------------- running a plan
    def _run(self, plan: StepPlan) -> None:
        try:
            with trace_range("scheduler.execute_batch"):
                sampled = self.runner.execute_batch(plan)
        except Exception as error:
            if not (_is_shortage(error) and self._make_room(error)):
                self._fail_plan(plan, error)
            return
        self._gave_way = False
        self._account(plan, sampled)

    def _start(self, plan: StepPlan) -> None:
        """Start a decode step without waiting for its tokens: no row has a token on the device yet."""
        placeholder = [-1] * len(plan.portions)
        next_index = [len(portion.request.output) for portion in plan.portions]
        try:
            with trace_range("scheduler.launch_decode"):
                handle = self._launch(plan, placeholder, next_index)
        except Exception as error:
            if not (_is_shortage(error) and self._make_room(error)):
                self._fail_plan(plan, error)
            return
        self._gave_way = False
        self._flying = _InFlight(plan, handle)

    def _fail_plan(self, plan: StepPlan, error: Exception) -> None:
        if _is_shortage(error):
            reason, rejected = f"KV capacity cannot fit one runnable sequence: {error}", True
        else:
            reason, rejected = f"packed forward failed: {error}", False
        for portion in plan.portions:
            if not portion.request.is_final:
                self._retire(portion.request, RequestState.FAILED, "failed", error=reason, rejected=rejected)

    def _account(self, plan: StepPlan, sampled: dict[str, int]) -> None:
        now = self.clock()
        for portion in plan.portions:
            request = portion.request
            if request.is_final:
                continue
            again = min(portion.end, request.redo_below) - portion.start
            if again > 0:
                request.recomputed += again
                self.metrics.totals.recomputed_tokens += again
            if not portion.samples:
                request.state = RequestState.PREFILL
            elif request.request_id in sampled:
                self._token_arrived(request, int(sampled[request.request_id]), now)
            else:
                self._retire(request, RequestState.FAILED, "failed", error="packed runner omitted sampled token")
        self.metrics.iteration(len(plan.portions), plan.token_count)

    def _token_arrived(self, request: Request, token: int, now: int) -> None:
        prompt_just_ended = request.state is RequestState.PREFILL
        request.output.append(token)
        if request.first_token_ns is None:
            request.first_token_ns = now
            self.metrics.first_token_ms.add((now - request.arrived_ns) * 1e-6)
        else:
            self.metrics.between_tokens_ms.add((now - request.latest_token_ns) * 1e-6)
        request.latest_token_ns = now
        self.metrics.totals.output_tokens += 1
        gen = request.gen
        if gen.eos_token_id is not None and token == gen.eos_token_id:
            # the id stays in ``output`` (ids are what a recomputation feeds) but is not streamed
            self._retire(request, RequestState.COMPLETED, "eos_token_reached")
            return
        if request.on_token is not None:
            request.on_token(request, token)
        if len(request.output) >= gen.max_output_tokens:
            self._retire(request, RequestState.COMPLETED, "max_output_tokens_reached")
            return
        request.state = RequestState.DECODING
        if prompt_just_ended and self._publish is not None:
            # the prompt's full pages will not change again: requests that arrive while this one
            # decodes may share them already
            self._publish(request)

    # ---------------------------------------------------------------- decode steps in flight
    def _collect(self) -> None:
        """Wait for the tokens of the step in flight and give them to their requests."""
        flying, self._flying = self._flying, None
        self._collecting = True
        try:
            self._account(flying.plan, flying.handle.tokens())
        finally:
            self._collecting = False

    def _follow_up(self, flying: StepPlan) -> tuple[StepPlan, list[int], list[int]] | None:
        """The step behind the one in flight, where it can be planned without that step's tokens:
        the same requests, less those whose token limit the token in flight reaches.  Row i takes
        its token from row ``feed[i]`` of the step in flight."""
        if self.waiting and len(self.active) < self.config.max_running:
            return None  # someone wants in: let the flight land, then admit
        aboard = {id(portion.request) for portion in flying.portions}
        if any(id(r) not in aboard for r in self.active if not r.is_final):
            return None  # someone has prompt left: the next step is a mixed one
        portions, feed, token_index = [], [], []
        for row, portion in enumerate(flying.portions):
            request = portion.request
            after_flight = len(request.output) + 1
            if request.is_final or after_flight >= request.gen.max_output_tokens:
                continue
            portions.append(Portion(request, request.cached, (0,), samples=True))
            feed.append(row)
            token_index.append(after_flight)
        if not portions or not self._launchable(len(portions)):
            return None
        return StepPlan(tuple(portions)), feed, token_index

    def _step_behind(self) -> None:
        follow = self._follow_up(self._flying.plan)
        handle = problem = None
        if follow is not None:
            try:
                with trace_range("scheduler.launch_decode"):
                    handle = self._launch(*follow)
            except Exception as error:  # nothing was started
                problem = error
        self._collect()
        if handle is not None:
            self._flying = _InFlight(follow[0], handle)
        elif problem is not None and not _is_shortage(problem):
            self._fail_plan(follow[0], problem)
        # a shortage is left alone here: the next call plans with every token in hand and makes room

    # ---------------------------------------------------------------- giving way and ending
    def _make_room(self, _error: Exception | None = None) -> bool:
        """Preempt one live request.  ``False`` if there is at most one, which then cannot run at all."""
        live = [r for r in self.active if not r.is_final]
        if len(live) < 2:
            return False
        resident = self._resident if self._resident is not None else (lambda _request: 0)
        victim = max(live, key=lambda r: self.victim_order(Standing.of(r, resident(r))))
        self.active.remove(victim)
        self._give_back(victim, preempted=True)
        victim.redo_below, victim.cached = victim.cached, 0
        victim.preemptions += 1
        victim.state = RequestState.WAITING
        self.waiting.appendleft(victim)
        self.metrics.totals.preempted += 1
        self._gave_way = True
        return True

    def _give_back(self, request: Request, preempted: bool = False) -> None:
        if self._release_knows_preemption:
            self.runner.release(request, preempted=preempted)
        else:
            self.runner.release(request)

    def _retire(self, request: Request, state: RequestState, reason: str, error: str = "",
                rejected: bool = False) -> None:
        """Every way a request ends passes here once: out of the queues, cache given back, counted."""
        if request.is_final:
            return
        request.state, request.finish_reason = state, reason
        request.error, request.rejected = error, rejected
        for queue in (self.active, self.waiting):
            if request in queue:
                queue.remove(request)
        try:
            self._give_back(request)
        except Exception as problem:  # an ending request must end, whatever the cache says
            request.error = f"release error: {problem}"
        request.ended_ns = self.clock()
        self.finished.append(request)
        totals = self.metrics.totals
        if state is RequestState.COMPLETED:
            totals.completed += 1
            self.metrics.whole_request_ms.add((request.ended_ns - request.arrived_ns) * 1e-6)
        elif state is RequestState.CANCELLED:
            totals.cancelled += 1
        elif rejected:
            totals.rejected += 1
        else:
            totals.failed += 1
