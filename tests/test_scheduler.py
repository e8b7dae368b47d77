"""CPU: the scheduler's decisions, with a fake runner in the manner of the
reference's tests/test_ragged_scheduler.py (FakePackedRunner :32-69: a token
capacity, a capacity error that carries ``is_capacity_error``, token
``100 + generated_count``)."""

import pytest

from cie_amd.config import build_engine_config
from cie_amd.engine.scheduler import (
    GenerationConfig, RejectedError, Refusal, RequestState, Scheduler,
)
from cie_amd.metrics import Metrics


class FakeRunner:
    def __init__(self, token_capacity: int = 10_000, eos_at: dict | None = None) -> None:
        self.token_capacity = token_capacity
        self.resident: dict[str, int] = {}
        self.traces: list[tuple[tuple[str, ...], tuple[int, ...]]] = []
        self.plans = []
        self.released: list[tuple[str, bool]] = []
        self.fail_next: Exception | None = None

    def admit(self, request) -> None:
        if request.request_id in self.resident:
            raise RuntimeError("duplicate admission")
        self.resident[request.request_id] = 0
        request.cached = 0

    def release(self, request, preempted: bool = False) -> None:
        if request.request_id in self.resident:
            self.released.append((request.request_id, preempted))
        self.resident.pop(request.request_id, None)

    def allocated_tokens(self, request) -> int:
        return self.resident.get(request.request_id, 0)

    def free_tokens(self) -> int:
        return self.token_capacity - sum(self.resident.values())

    def execute_batch(self, plan):
        if self.fail_next is not None:
            error, self.fail_next = self.fail_next, None
            raise error
        required = dict(self.resident)
        for item in plan.portions:
            required[item.request.request_id] = max(required[item.request.request_id], item.end)
        if sum(required.values()) > self.token_capacity:
            error = RuntimeError("fake KV capacity exhausted")
            error.is_capacity_error = True
            raise error
        self.resident = required
        self.plans.append(plan)
        self.traces.append((plan.request_ids, tuple(item.length for item in plan.portions)))
        outputs = {}
        for item in plan.portions:
            assert item.start == item.request.cached, "a portion must start where the cache ends"
            item.request.cached = item.end
            if item.samples:
                outputs[item.request.request_id] = 100 + len(item.request.output)
        return outputs


def make(runner, **overrides):
    # (the fake runners count tokens, not pages: a page of one token)
    options = dict(max_model_len=128, max_running=4, max_queue_size=8, token_budget=16, prefill_chunk=4, page_size=1)
    options.update(overrides)
    return Scheduler(build_engine_config(**options), runner, Metrics())


def test_requests_share_one_forward():
    runner = FakeRunner()
    scheduler = make(runner)
    requests = [scheduler.submit([i + 1] * 3, GenerationConfig(max_output_tokens=2)) for i in range(3)]
    scheduler.run_until_done(100)
    assert [r.output for r in requests] == [[100, 101]] * 3
    assert any(len(ids) == 3 for ids, _ in runner.traces)
    assert all(r.state is RequestState.COMPLETED and r.finish_reason == "max_output_tokens_reached" for r in requests)
    assert not runner.resident


def test_prefill_is_cut_into_portions_under_the_budget():
    runner = FakeRunner()
    scheduler = make(runner, token_budget=5, prefill_chunk=4)
    request = scheduler.submit(list(range(11)), GenerationConfig(max_output_tokens=1))
    scheduler.run_until_done(100)
    assert request.output == [100]
    assert [lengths[0] for _, lengths in runner.traces][:3] == [4, 4, 3]
    samples = [item.samples for plan in runner.plans for item in plan.portions]
    assert samples == [False, False, True]  # logits only where the portion reaches the tail


def test_decode_goes_first_and_budget_is_shared():
    runner = FakeRunner()
    scheduler = make(runner, token_budget=6, prefill_chunk=4)
    first = scheduler.submit([1] * 2, GenerationConfig(max_output_tokens=4))
    scheduler.step()  # first: whole prompt, gets a token, now decoding
    late = scheduler.submit([2] * 20, GenerationConfig(max_output_tokens=1))
    scheduler.step()
    plan = runner.plans[-1]
    assert plan.request_ids == (first.request_id, late.request_id)
    assert [item.length for item in plan.portions] == [1, 4] and plan.portions[0].is_decode
    assert not plan.portions[1].is_decode and plan.token_count <= 6
    scheduler.run_until_done(100)
    for plan in runner.plans:
        assert plan.token_count <= 6 and len(set(plan.request_ids)) == len(plan.request_ids)
        phases = [item.is_decode for item in plan.portions]
        assert phases == sorted(phases, reverse=True), "decode items come before prefill items"


def test_custom_priority_reorders_but_cannot_exceed_budget():
    runner = FakeRunner()
    scheduler = make(runner, token_budget=4)
    scheduler.plan_order = lambda standing: (standing.pending_tokens,)
    long = scheduler.submit([1] * 8, GenerationConfig(max_output_tokens=1))
    short = scheduler.submit([2] * 2, GenerationConfig(max_output_tokens=1))
    scheduler._admit()
    plan = scheduler._plan()
    assert plan.request_ids == (short.request_id, long.request_id) and plan.token_count == 4


def test_pressure_preempts_then_recomputes_without_token_drift():
    runner = FakeRunner(token_capacity=10)
    scheduler = make(runner, token_budget=8, prefill_chunk=4)
    requests = [scheduler.submit([i + 1] * 4, GenerationConfig(max_output_tokens=3)) for i in range(2)]
    scheduler.run_until_done(200)
    assert [r.output for r in requests] == [[100, 101, 102]] * 2
    assert sum(r.preemptions for r in requests) > 0 and sum(r.recomputed for r in requests) > 0
    snapshot = scheduler.metrics.snapshot()
    assert snapshot["requests"]["preempted_total"] > 0 and snapshot["tokens"]["recomputed_total"] > 0
    assert snapshot["requests"]["completed_total"] == 2
    assert not runner.resident
    assert any(flag for _, flag in runner.released), "a preemption releases without storing a prefix"


def test_preempted_request_keeps_generated_tokens_and_its_place():
    runner = FakeRunner(token_capacity=12)
    scheduler = make(runner, token_budget=16, prefill_chunk=8)
    a = scheduler.submit([1] * 5, GenerationConfig(max_output_tokens=4))
    b = scheduler.submit([2] * 5, GenerationConfig(max_output_tokens=4))
    c = scheduler.submit([3] * 2, GenerationConfig(max_output_tokens=1))
    scheduler.config = build_engine_config(scheduler.config, max_running=2)
    scheduler.step()  # a and b prefilled: 10 resident; each has its first token
    scheduler.step()  # 12 resident
    assert (len(a.output), len(b.output)) == (2, 2)
    scheduler.step()  # 14 > 12: the larger one (tie: the later arrival) is preempted
    assert b.state is RequestState.WAITING and b.preemptions == 1 and b.cached == 0
    assert b.output == [100, 101] and b.redo_below == 6
    assert scheduler.waiting[0] is b, "the preempted request waits at the head, before the newcomer"
    scheduler.step()  # a decodes alone: 7 resident, 5 free; b needs 5 + 2 + 1 = 8: still waiting, c behind it
    assert b.state is RequestState.WAITING and c.state is RequestState.WAITING
    scheduler.run_until_done(200)
    assert [r.output for r in (a, b, c)] == [[100, 101, 102, 103]] * 2 + [[100]]
    # the recompute fed prompt and generated tokens as prompt portions and sampled only at the tail
    recompute = [item for plan in runner.plans for item in plan.portions
                 if item.request is b and item.start == 0 and item.length > 5]
    assert recompute and recompute[0].tokens == (2, 2, 2, 2, 2, 100, 101) and recompute[0].samples


def test_long_prompts_are_admitted_only_while_the_pool_holds_them():
    """Three prompts of which the pool holds two: the third waits until one has
    ended, nothing is preempted and nothing computed twice; admitted as the
    reference admits (without a look at the pool) they push each other out."""
    def run(admit_within_pool):
        runner = FakeRunner(token_capacity=24)
        scheduler = make(runner, token_budget=8, prefill_chunk=4, admit_within_pool=admit_within_pool)
        requests = [scheduler.submit([i + 1] * 9, GenerationConfig(max_output_tokens=2)) for i in range(3)]
        scheduler.step()
        admitted = len(scheduler.active)
        scheduler.run_until_done(200)
        assert [r.output for r in requests] == [[100, 101]] * 3 and not runner.resident
        return admitted, sum(r.preemptions for r in requests), sum(r.recomputed for r in requests)

    assert run(True) == (2, 0, 0)
    admitted, preempted, recomputed = run(False)
    assert admitted == 3 and preempted > 0 and recomputed > 0


def test_a_request_larger_than_what_is_left_is_admitted_when_nothing_else_runs():
    runner = FakeRunner(token_capacity=12)
    scheduler = make(runner, token_budget=16, prefill_chunk=16)
    first = scheduler.submit([1] * 8, GenerationConfig(max_output_tokens=2))
    second = scheduler.submit([2] * 8, GenerationConfig(max_output_tokens=2))
    scheduler.step()
    assert [r.request_id for r in scheduler.active] == [first.request_id] and scheduler.waiting[0] is second
    scheduler.run_until_done(100)
    assert first.output == second.output == [100, 101]
    assert first.preemptions == second.preemptions == 0


def test_over_subscribed_pools_drain_under_random_loads():
    """Thirty requests through pools that hold a few of them, under random budgets,
    portions, limits of running requests and both ways of admission: every request
    ends, with the tokens it would have had alone.  (A preempted request that was taken
    back as soon as the pages it had just returned were free took them from the same
    requests again, for ever: 36 of these 300 loads did not end.)"""
    import random

    for seed in range(300):
        rng = random.Random(seed)
        runner = FakeRunner(token_capacity=rng.randint(30, 80))
        scheduler = make(runner, token_budget=rng.choice([8, 16, 64]), prefill_chunk=rng.choice([3, 8, 16]),
                         admit_within_pool=rng.random() < 0.5, max_running=rng.choice([2, 4, 8, 16]), max_queue_size=100)
        requests = [scheduler.submit([i + 1] * rng.randint(1, 12), GenerationConfig(max_output_tokens=rng.randint(1, 12)))
                    for i in range(30)]
        scheduler.run_until_done(5000)
        for request in requests:
            assert request.state is RequestState.COMPLETED, (seed, request.state, request.error)
            assert request.output == [100 + i for i in range(request.gen.max_output_tokens)], seed
        assert not runner.resident, seed


def test_custom_preemption_policy_selects_victim():
    runner = FakeRunner(token_capacity=10)
    scheduler = make(runner, token_budget=8, prefill_chunk=4)
    scheduler.victim_order = lambda standing: (-standing.arrived_ns,)
    requests = [scheduler.submit([i + 1] * 4, GenerationConfig(max_output_tokens=3)) for i in range(2)]
    scheduler._admit()
    runner.resident = {r.request_id: 4 for r in requests}
    assert scheduler._make_room()
    assert (requests[0].preemptions, requests[1].preemptions) == (1, 0)


def test_single_request_that_cannot_fit_is_rejected():
    runner = FakeRunner(token_capacity=6)
    scheduler = make(runner, token_budget=16, prefill_chunk=16)
    request = scheduler.submit([1] * 8, GenerationConfig(max_output_tokens=2))
    scheduler.run_until_done(10)
    assert request.state is RequestState.FAILED and request.rejected
    assert "KV capacity cannot fit one runnable sequence" in request.error
    assert scheduler.metrics.snapshot()["requests"]["rejected_total"] == 1 and not runner.resident


def test_submit_time_rejections():
    scheduler = make(FakeRunner(), max_queue_size=2, max_model_len=16)
    with pytest.raises(RejectedError) as caught:
        scheduler.submit([], GenerationConfig(max_output_tokens=1))
    assert caught.value.reason is Refusal.TOO_LONG
    with pytest.raises(RejectedError) as caught:
        scheduler.submit([1] * 10, GenerationConfig(max_output_tokens=7))
    assert caught.value.reason is Refusal.TOO_LONG
    scheduler.submit([1] * 10, GenerationConfig(max_output_tokens=6))
    scheduler.submit([1], GenerationConfig(max_output_tokens=1))
    with pytest.raises(RejectedError) as caught:
        scheduler.submit([1], GenerationConfig(max_output_tokens=1))
    assert caught.value.reason is Refusal.QUEUE_FULL
    assert [r.request_id for r in scheduler.waiting] == ["req-00000001", "req-00000002"]


def test_generation_config_validation():
    assert GenerationConfig(max_output_tokens=1, temperature=0.8).temperature == 0.8
    with pytest.raises(ValueError):
        GenerationConfig(max_output_tokens=1, temperature=-1.0)
    with pytest.raises(ValueError):
        GenerationConfig(max_output_tokens=0)


def test_eos_finishes_and_is_kept_but_not_streamed():
    runner = FakeRunner()
    scheduler = make(runner)
    streamed = []
    request = scheduler.submit([1, 2], GenerationConfig(max_output_tokens=10, eos_token_id=102),
                               on_token=lambda r, t: streamed.append(t))
    ignoring = scheduler.submit([1, 2], GenerationConfig(max_output_tokens=4, eos_token_id=None))
    scheduler.run_until_done(100)
    assert request.output == [100, 101, 102] and request.finish_reason == "eos_token_reached"
    assert streamed == [100, 101]
    assert ignoring.output == [100, 101, 102, 103]


def test_active_limit_and_fifo_admission():
    runner = FakeRunner()
    scheduler = make(runner, max_running=2)
    requests = [scheduler.submit([1] * 2, GenerationConfig(max_output_tokens=2)) for _ in range(4)]
    scheduler.step()
    assert [r.state for r in requests[:2]] == [RequestState.DECODING] * 2
    assert [r.state for r in requests[2:]] == [RequestState.WAITING] * 2
    scheduler.run_until_done(100)
    assert max(len(ids) for ids, _ in runner.traces) == 2
    order = [rid for rid, _ in runner.released]
    assert order == [r.request_id for r in requests]


def test_cancel_is_idempotent_and_frees():
    runner = FakeRunner()
    scheduler = make(runner)
    request = scheduler.submit([1] * 3, GenerationConfig(max_output_tokens=5))
    waiting = scheduler.submit([1] * 3, GenerationConfig(max_output_tokens=5))
    scheduler.step()
    scheduler.cancel(request)
    scheduler.cancel(request)
    scheduler.cancel(waiting)
    assert request.state is RequestState.CANCELLED and not runner.resident and not scheduler.has_work()
    assert scheduler.metrics.snapshot()["requests"]["cancelled_total"] == 2


def test_forward_failure_fails_the_plan_and_the_loop_goes_on():
    runner = FakeRunner()
    scheduler = make(runner)
    doomed = scheduler.submit([1] * 3, GenerationConfig(max_output_tokens=2))
    runner.fail_next = RuntimeError("kernel exploded")
    scheduler.step()
    assert doomed.state is RequestState.FAILED and not doomed.rejected and "kernel exploded" in doomed.error
    later = scheduler.submit([1] * 3, GenerationConfig(max_output_tokens=2))
    scheduler.run_until_done(100)
    assert later.output == [100, 101] and not runner.resident


def test_admission_failure_is_counted():
    class Refusing(FakeRunner):
        def admit(self, request):
            error = RuntimeError("no slot")
            error.is_capacity_error = True
            raise error

    scheduler = make(Refusing())
    request = scheduler.submit([1], GenerationConfig(max_output_tokens=1))
    scheduler.step()
    assert request.state is RequestState.FAILED and request.rejected and "admission refused" in request.error


def test_prompt_is_published_once_its_last_portion_has_run():
    """A runner that can publish prefixes is told when a request's prompt is all in
    the cache (at its first token), again after a recomputation, and not for a
    request that ends with its first token."""
    class Publishing(FakeRunner):
        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            self.published = []

        def publish_prefix(self, request) -> None:
            assert request.cached >= len(request.prompt)
            self.published.append((request.request_id, len(request.output)))

    runner = Publishing()
    scheduler = make(runner)
    long_one = scheduler.submit(list(range(9)), GenerationConfig(max_output_tokens=3))
    one_token = scheduler.submit(list(range(5)), GenerationConfig(max_output_tokens=1))
    scheduler.run_until_done()
    assert runner.published == [(long_one.request_id, 1)]
    assert one_token.state is RequestState.COMPLETED


# -- decode steps that are started before the tokens of the step before have arrived ----------------
class AsyncFakeRunner(FakeRunner):
    """A fake with ``launch_decode``: tokens come back through a pending object that counts how often it
    was waited for; a fed row's token is what the launch before produced (kept "on the device")."""

    def __init__(self, *args, eos_token_at=None, **kwargs):
        super().__init__(*args, **kwargs)
        self.launches: list[tuple[tuple[str, ...], tuple[int, ...]]] = []
        self.device_tokens: list[int] = []
        self.eos_token_at = eos_token_at or {}  # request serial -> (token index, token id)

    def can_launch_decode(self, requests: int) -> bool:
        return requests <= 8

    def _token(self, request, index: int) -> int:
        at = self.eos_token_at.get(request.serial)
        return at[1] if at is not None and at[0] == index else 100 + index

    def execute_batch(self, plan):
        outputs = super().execute_batch(plan)
        return {item.request.request_id: self._token(item.request, len(item.request.output))
                for item in plan.portions if item.request.request_id in outputs}

    def launch_decode(self, plan, feed, token_indices):
        required = dict(self.resident)
        for item in plan.portions:
            required[item.request.request_id] = max(required[item.request.request_id], item.end)
        if sum(required.values()) > self.token_capacity:
            error = RuntimeError("fake KV capacity exhausted")
            error.is_capacity_error = True
            raise error
        self.resident = required
        fed_tokens = []
        for item, source in zip(plan.portions, feed):
            assert item.start == item.request.cached and item.length == 1
            fed_tokens.append(self.device_tokens[source] if source >= 0 else item.tokens[0])
            item.request.cached = item.end
        self.launches.append((plan.request_ids, tuple(fed_tokens)))
        self.device_tokens = [self._token(item.request, index) for item, index in zip(plan.portions, token_indices)]
        produced = dict(zip(plan.request_ids, self.device_tokens))

        class Pending:
            def tokens(_self):
                return produced

        return Pending()


def make_async(runner, **overrides):
    return make(runner, async_decode=True, **overrides)


def test_async_decode_gives_the_same_tokens_with_one_launch_per_token():
    def run(scheduler_of):
        runner = AsyncFakeRunner()
        scheduler = scheduler_of(runner)
        a = scheduler.submit(list(range(6)), GenerationConfig(max_output_tokens=5))
        b = scheduler.submit(list(range(3)), GenerationConfig(max_output_tokens=3))
        scheduler.run_until_done()
        return runner, a, b

    sync_runner, a0, b0 = run(lambda r: make(r, async_decode=False))
    runner, a, b = run(make_async)
    assert not sync_runner.launches and runner.launches
    assert a.output == a0.output == [100, 101, 102, 103, 104]
    assert b.output == b0.output == [100, 101, 102]
    # the first token of each comes with its prompt; every further token is one row of one launch, no more:
    # b leaves the launches when its limit is in sight, nothing runs for a token that is not wanted
    launched_rows = sum(len(ids) for ids, _ in runner.launches)
    sampled_with_prompts = sum(item.samples for plan in runner.plans for item in plan.portions)
    assert launched_rows + sampled_with_prompts == 5 + 3
    # from the second launch on, rows are fed the token the launch before made, not a placeholder
    assert runner.launches[1][1][0] == 101
    assert a.state is RequestState.COMPLETED and b.state is RequestState.COMPLETED and not runner.resident


def test_async_decode_tokens_arrive_one_call_late():
    runner = AsyncFakeRunner()
    scheduler = make_async(runner)
    request = scheduler.submit(list(range(4)), GenerationConfig(max_output_tokens=6))
    scheduler.step()                    # the prompt, with its first token
    assert len(request.output) == 1
    scheduler.step()                    # launches token 2; nothing has arrived
    assert len(request.output) == 1 and scheduler.has_work()
    scheduler.step()                    # launches token 3, takes token 2
    assert len(request.output) == 2
    scheduler.run_until_done()
    assert request.output == [100, 101, 102, 103, 104, 105]


def test_async_decode_end_of_sequence_costs_one_dropped_step():
    runner = AsyncFakeRunner(eos_token_at={1: (2, 7)})  # the first request's third token is token 7
    scheduler = make_async(runner)
    stops = scheduler.submit(list(range(4)), GenerationConfig(max_output_tokens=10, eos_token_id=7))
    goes_on = scheduler.submit(list(range(4)), GenerationConfig(max_output_tokens=6))
    scheduler.run_until_done()
    assert stops.output == [100, 101, 7] and stops.finish_reason == "eos_token_reached"
    assert goes_on.output == [100, 101, 102, 103, 104, 105]
    launched_for_stops = sum(stops.request_id in ids for ids, _ in runner.launches)
    assert launched_for_stops == 3  # tokens 2 and 3, and one step more that was under way when token 7 arrived
    assert not runner.resident and (stops.request_id, False) in runner.released


def test_async_decode_lets_a_new_request_in_and_survives_a_shortage():
    runner = AsyncFakeRunner(token_capacity=30)
    scheduler = make_async(runner, max_running=3)
    first = scheduler.submit(list(range(8)), GenerationConfig(max_output_tokens=12))
    for _ in range(4):
        scheduler.step()
    late = scheduler.submit(list(range(8)), GenerationConfig(max_output_tokens=12))  # both need 20: one must wait
    scheduler.run_until_done(max_iterations=200)
    assert first.output == [100 + i for i in range(12)]
    assert late.output == [100 + i for i in range(12)]
    assert scheduler.metrics.snapshot()["requests"]["preempted_total"] >= 1
    assert not runner.resident


def test_async_decode_cancel_takes_what_is_in_flight_first():
    runner = AsyncFakeRunner()
    scheduler = make_async(runner)
    request = scheduler.submit(list(range(4)), GenerationConfig(max_output_tokens=9))
    for _ in range(3):
        scheduler.step()
    assert len(request.output) == 2
    scheduler.cancel(request)
    assert request.state is RequestState.CANCELLED and len(request.output) == 3 and not scheduler.has_work()
    assert not runner.resident


# -- a runner that keeps a real cache manager (no tensors): what admission sees of the pool -------------
class ManagerRunner:
    def __init__(self, manager) -> None:
        self.cache = manager
        self.most_side_by_side = 0

    def admit(self, request) -> None:
        request.cached = self.cache.admit(request.request_id, request.prompt)

    def release(self, request, preempted: bool = False) -> None:
        self.cache.release(request.request_id, None if preempted else request.prompt)

    def allocated_tokens(self, request) -> int:
        return self.cache.allocated_tokens(request.request_id)

    def free_tokens(self) -> int:
        return self.cache.free_tokens()

    def tokens_needed(self, request, upto: int) -> int:
        return self.cache.tokens_missing(request.request_id, upto)

    def execute_batch(self, plan):
        need = {p.request.request_id: p.end for p in plan.portions}
        self.cache.ensure_capacity_batch(need)
        self.cache.commit_lengths(need)
        self.most_side_by_side = max(self.most_side_by_side, len(plan.portions))
        for portion in plan.portions:
            portion.request.cached = portion.end
        return {p.request.request_id: 100 + len(p.request.output) for p in plan.portions if p.samples}


def test_pages_that_only_the_prefix_index_holds_do_not_block_admission():
    """Earlier requests have left the index full; the free list alone holds one newcomer.  The
    newcomers still run side by side: what the index holds alone is evicted when they grow."""
    from cie_amd.cache.manager import CacheManager, PagedKV

    manager = CacheManager([PagedKV(1, 8)], page_size=4, kv_tokens=64, max_running=8, max_model_len=64,
                           prefix_cache_pages=12)
    runner = ManagerRunner(manager)
    scheduler = make(runner, max_model_len=64, max_running=8, token_budget=64, prefill_chunk=16, page_size=4)
    for i in range(3):  # three prompts of 17 tokens leave four full pages each
        scheduler.submit([i + 1] * 17, GenerationConfig(max_output_tokens=1))
    scheduler.run_until_done(50)
    assert manager.stats().prefix_pages_used == 12 and manager.groups[0].allocator.free_count == 4
    runner.most_side_by_side = 0
    fresh = [scheduler.submit([50 + i] * 9, GenerationConfig(max_output_tokens=3)) for i in range(4)]
    scheduler.run_until_done(50)
    assert runner.most_side_by_side == 4, "each needs 3 pages; 4 are free, 12 more can be evicted"
    assert all(r.output == [100, 101, 102] and r.preemptions == 0 for r in fresh)
    manager.assert_invariants()


def test_a_cache_without_pages_admits_side_by_side():
    """Every unit a state of fixed size: nothing is paged, so the pool never makes a request wait."""
    from cie_amd.cache.manager import CacheManager, FixedState

    runner = ManagerRunner(CacheManager([FixedState((4,))], page_size=4, kv_tokens=4, max_running=4, max_model_len=64))
    scheduler = make(runner, max_model_len=64, max_running=4, admit_within_pool=True)
    requests = [scheduler.submit([i + 1] * 6, GenerationConfig(max_output_tokens=4)) for i in range(4)]
    scheduler.step()
    assert len(scheduler.active) == 4
    scheduler.run_until_done(50)
    assert runner.most_side_by_side == 4 and all(r.output == [100, 101, 102, 103] for r in requests)


def test_admission_asks_the_runner_what_a_request_costs():
    """A cache whose only group keeps a window of 8 keys: a request of 40 tokens never holds more than four
    pages of 4, so four of them run side by side in a pool of 16 pages, which by their length alone
    (11 pages each) would hold one.  The scheduler takes the cost from the runner, not from the page size."""
    from cie_amd.cache.manager import CacheManager, PagedKV

    manager = CacheManager([PagedKV(1, 8, window=8)], page_size=4, kv_tokens=64, max_running=4, max_model_len=64,
                           prefill_chunk=4)
    assert manager.groups[0].allocator.total_pages == 16 and manager.groups[0].most_per_request == 4
    assert manager.tokens_missing("nobody", 41) == 16 and manager.tokens_missing("nobody", 5) == 8
    runner = ManagerRunner(manager)
    scheduler = make(runner, max_model_len=64, max_running=4, token_budget=16, prefill_chunk=4, page_size=4,
                     admit_within_pool=True)
    requests = [scheduler.submit([i + 1] * 40, GenerationConfig(max_output_tokens=3)) for i in range(4)]
    scheduler.step()
    assert len(scheduler.active) == 4
    scheduler.run_until_done(200)
    assert runner.most_side_by_side == 4 and all(r.output == [100, 101, 102] and r.preemptions == 0 for r in requests)
    manager.assert_invariants()
    # a runner that does not say falls back on whole pages per token: one request at a time here
    silent = ManagerRunner(CacheManager([PagedKV(1, 8, window=8)], page_size=4, kv_tokens=64, max_running=4,
                                        max_model_len=64, prefill_chunk=4))
    silent.tokens_needed = None
    scheduler = make(silent, max_model_len=64, max_running=4, token_budget=16, prefill_chunk=4, page_size=4,
                     admit_within_pool=True)
    for i in range(4):
        scheduler.submit([i + 1] * 40, GenerationConfig(max_output_tokens=3))
    scheduler.step()
    assert len(scheduler.active) == 1


@pytest.mark.parametrize("seed", [3, 12, 21, 30])
def test_pools_of_whole_pages_drain_under_random_loads(seed):
    """Random prompts (half of them behind a common prefix), output lengths and arrivals through the real cache
    manager with a pool of a few pages, a prefix index and both ways of admission.  A request takes whole pages, so
    the room that admission reckons with has to be reckoned in pages, and a request that has just given way must
    not come back before the others have run: else it is let in, the step fails for want of a page, it gives way
    again, and nothing ever runs (seed 12 did exactly that, 1,883 times over, before this was seen to)."""
    import random

    from cie_amd.cache.manager import CacheManager, PagedKV

    rng = random.Random(seed)
    limit, vocab = 128, 256
    prefix = [rng.randrange(vocab) for _ in range(40)]
    requests = []
    for _ in range(60):
        n = rng.randint(1, limit // 2)
        prompt = prefix[: rng.randint(0, min(40, n - 1))] if rng.random() < 0.5 and n > 1 else []
        prompt = prompt + [rng.randrange(vocab) for _ in range(n - len(prompt))]
        out = rng.randint(1, min(40, limit - n - 1))
        rng.choice([0.0, 0.0, 0.7, 1.3])
        requests.append((prompt, GenerationConfig(max_output_tokens=out, eos_token_id=rng.choice([None, None, rng.randrange(vocab)]))))
        rng.randrange(1000)
    page, running = rng.choice([4, 8, 16]), rng.choice([4, 8, 16])
    budget, chunk, within = rng.choice([32, 64, 256]), rng.choice([7, 16, 64]), rng.random() < 0.5
    manager = CacheManager([PagedKV(2, 16)], page_size=page, kv_tokens=3 * limit, max_running=running, max_model_len=limit,
                           prefix_cache_pages=16)
    runner = ManagerRunner(manager)
    runner.publish_prefix = lambda request: manager.publish_prefix(request.request_id, request.prompt)
    scheduler = make(runner, page_size=page, kv_tokens=3 * limit, max_running=running, max_queue_size=100, max_model_len=limit,
                     max_output_tokens=64, token_budget=budget, prefill_chunk=chunk, prefix_cache_pages=16,
                     admit_within_pool=within)
    handles, pending, steps = [], list(requests), 0
    while pending or scheduler.has_work():
        for _ in range(rng.randint(0, 3)):
            if pending:
                prompt, gen = pending.pop(0)
                handles.append(scheduler.submit(prompt, gen))
        scheduler.step()
        steps += 1
        assert steps < 2000, ("the scheduler does not drain", page, running, budget, chunk, within,
                              [(r.state.value, r.cached, r.preemptions) for r in scheduler.active])
    assert all(h.state is RequestState.COMPLETED for h in handles)
    assert all(len(h.output) == h.gen.max_output_tokens or h.finish_reason == "eos_token_reached" for h in handles)
    manager.assert_invariants()
    assert manager.stats().pages_used == manager.stats().prefix_pages_used
