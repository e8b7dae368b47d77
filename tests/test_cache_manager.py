"""CPU: page allocator and cache manager.  The allocator cases are those of the
reference's tests/test_allocator.py (values at :12-18, exhaustion :29-37, reuse
:39-44, double/foreign/duplicate free :46-64, churn :66-91, single owner :93-97)."""

import random

import pytest

from cie_amd.cache import (
    PREFIX_HOLDER, CacheCapacityFull, CacheManager, DoubleFreeError, FixedState, PageAllocator, PagedKV,
)


# -- allocator -----------------------------------------------------------------------
def test_pages_for_rounds_up():
    allocator = PageAllocator(8, 16)
    assert [allocator.pages_for(n) for n in (0, 1, 15, 16, 17, 2048)] == [0, 1, 1, 1, 2, 128]


def test_allocate_free_roundtrip_and_exhaustion():
    allocator = PageAllocator(8, 16)
    pages = allocator.allocate("req-a", 3)
    assert (len(pages), allocator.used_count, allocator.free_count) == (3, 3, 5)
    allocator.free(pages, "req-a")
    assert (allocator.used_count, allocator.free_count) == (0, 8)
    with pytest.raises(CacheCapacityFull):
        allocator.allocate("req-big", 9)
    exact = allocator.allocate("req-exact", 8)
    with pytest.raises(CacheCapacityFull) as caught:
        allocator.allocate("req-one-more", 1)
    assert caught.value.is_capacity_error
    allocator.free(exact, "req-exact")


def test_freed_pages_are_used_again_most_recent_first():
    allocator = PageAllocator(8, 16)
    first = allocator.allocate("req-a", 2)
    allocator.free(first, "req-a")
    second = allocator.allocate("req-b", 2)
    assert set(first) == set(second)


def test_double_foreign_and_duplicate_free():
    allocator = PageAllocator(8, 16)
    pages = allocator.allocate("req-a", 2)
    with pytest.raises(DoubleFreeError):
        allocator.free(pages, "req-b")
    assert allocator.held_by("req-a") == 2  # a failed free changes nothing
    with pytest.raises(DoubleFreeError):
        allocator.free([pages[0], pages[0]], "req-a")
    with pytest.raises(DoubleFreeError):
        allocator.free([pages[0], 7], "req-a")  # 7 is free; pages[0] must stay held
    assert allocator.held_by("req-a") == 2
    allocator.free(pages, "req-a")
    with pytest.raises(DoubleFreeError):
        allocator.free(pages, "req-a")


def test_invariants_hold_through_churn():
    allocator = PageAllocator(8, 16)
    live: dict[str, list[int]] = {}
    rng = random.Random(7)
    serial = 0
    for _ in range(500):
        if live and rng.random() < 0.45:
            owner = rng.choice(list(live))
            count = min(rng.randint(1, 3), len(live[owner]))
            released, live[owner] = live[owner][:count], live[owner][count:]
            allocator.free(released, owner)
            if not live[owner]:
                del live[owner]
        else:
            try:
                live[f"req-{serial}"] = allocator.allocate(f"req-{serial}", rng.randint(1, 4))
                serial += 1
            except CacheCapacityFull:
                pass
        allocator.assert_invariants()
        held = [p for pages in live.values() for p in pages]
        assert len(held) == len(set(held)), "a page has two owners"
        assert allocator.used_count == len(held) and allocator.used_count + allocator.free_count == 8


def test_shared_page_returns_when_last_holder_lets_go():
    allocator = PageAllocator(4, 16)
    (page,) = allocator.allocate("a", 1)
    allocator.retain(page, "b")
    with pytest.raises(DoubleFreeError):
        allocator.retain(page, "b")
    assert allocator.free([page], "a") == [] and allocator.used_count == 1
    assert allocator.free([page], "b") == [page] and allocator.free_count == 4
    with pytest.raises(DoubleFreeError):
        allocator.retain(page, "c")


# -- manager -------------------------------------------------------------------------
def manager(**kw):
    defaults = dict(unit_specs=[PagedKV(2, 16)] * 2, page_size=4, kv_tokens=64, max_running=4, max_model_len=64)
    defaults.update(kw)
    return CacheManager(**defaults)


def test_growth_is_all_or_nothing():
    m = manager(kv_tokens=32)  # 8 pages
    m.admit("a"), m.admit("b")
    m.ensure_capacity_batch({"a": 9, "b": 4})
    assert len(m.block_table(0, "a")) == 3 and len(m.block_table(0, "b")) == 1
    before = (m.block_table(0, "a"), m.block_table(0, "b"), m.stats().pages_used)
    with pytest.raises(CacheCapacityFull):
        m.ensure_capacity_batch({"a": 12, "b": 24})  # needs 0 + 5 more, 4 free
    assert (m.block_table(0, "a"), m.block_table(0, "b"), m.stats().pages_used) == before
    m.ensure_capacity_batch({"b": 20})  # exactly the 4 free pages
    assert m.stats().pages_used == 8
    with pytest.raises(KeyError):
        m.ensure_capacity_batch({"nobody": 1})
    with pytest.raises(ValueError, match="max_model_len"):
        m.ensure_capacity_batch({"a": 65})
    m.assert_invariants()


def test_commit_checks_pages_and_release_returns_everything():
    m = manager()
    m.admit("a")
    with pytest.raises(RuntimeError, match="exceeds allocated"):
        m.commit_lengths({"a": 5})
    m.ensure_capacity_batch({"a": 5})
    m.commit_lengths({"a": 5})
    assert m.length("a") == 5 and m.allocated_tokens("a") == 8
    m.release("a")
    m.release("a")  # idempotent
    assert m.stats().pages_used == 0 and m.stats().slots_used == 0 and not m.has("a")
    m.assert_invariants()


def test_slots_are_taken_and_given_back():
    m = manager(max_running=2)
    assert m.admit("a") == 0 and m.admit("b") == 0
    assert {m.slot("a"), m.slot("b")} == {0, 1}
    with pytest.raises(CacheCapacityFull, match="slots"):
        m.admit("c")
    with pytest.raises(ValueError, match="duplicate"):
        m.admit("a")
    freed = m.slot("a")
    m.release("a")
    m.admit("c")
    assert m.slot("c") == freed
    assert sorted(m.take_fresh_slots()) == [0, 1]
    assert m.take_fresh_slots() == []


def test_pages_of_a_finished_request_are_used_again():
    m = manager(kv_tokens=16)  # 4 pages
    m.admit("a")
    m.ensure_capacity_batch({"a": 16})
    pages = m.block_table(0, "a")
    m.admit("b")
    with pytest.raises(CacheCapacityFull):
        m.ensure_capacity_batch({"b": 1})
    m.release("a")
    m.ensure_capacity_batch({"b": 16})
    assert set(m.block_table(0, "b")) == set(pages)


def test_dirty_rows_follow_table_changes():
    m = manager()
    m.admit("a")
    assert m.take_dirty_rows() == [(0, m.slot("a"), [])]
    m.ensure_capacity_batch({"a": 4})
    m.ensure_capacity_batch({"a": 4})  # no growth, not dirty again
    rows = m.take_dirty_rows()
    assert rows == [(0, m.slot("a"), m.block_table(0, "a"))] and m.take_dirty_rows() == []


def test_random_request_orders_lose_no_page():
    rng = random.Random(3)
    m = manager(kv_tokens=128, max_running=5, max_model_len=48, prefix_cache_pages=6,
                unit_specs=[PagedKV(2, 16)] * 3)
    live: dict[str, tuple[list[int], int]] = {}
    serial = 0
    for _ in range(1500):
        roll = rng.random()
        if roll < 0.25 and len(live) < 5:
            prompt = [rng.randrange(3) for _ in range(rng.randint(1, 30))]  # tiny alphabet: prefixes collide
            rid = f"r{serial}"
            serial += 1
            reused = m.admit(rid, prompt)
            assert reused % 4 == 0 and reused < len(prompt)
            live[rid] = (prompt, reused)
        elif roll < 0.8 and live:
            rid = rng.choice(list(live))
            prompt, fed = live[rid]
            target = min(48, fed + rng.randint(1, 9))
            try:
                m.ensure_capacity_batch({rid: target})
                m.commit_lengths({rid: target})
                live[rid] = (prompt, target)
            except CacheCapacityFull:
                victim = max(live, key=lambda r: m.allocated_tokens(r))
                m.release(victim)  # preemption: no prefix stored
                del live[victim]
        elif live:
            rid = rng.choice(list(live))
            m.release(rid, live.pop(rid)[0])
        m.assert_invariants()
        stats = m.stats()
        assert stats.prefix_pages_used <= 6 and stats.slots_used == len(live)
    for rid in list(live):
        m.release(rid)
    m.clear_prefix_index()
    m.assert_invariants()
    assert m.stats().pages_used == 0


# -- windows and fixed state -----------------------------------------------------------
def test_window_group_gives_pages_back_as_the_window_passes():
    m = manager(unit_specs=[PagedKV(2, 16), PagedKV(2, 16, window=6), PagedKV(2, 16, window=6)],
                kv_tokens=64, prefill_chunk=8)
    assert len(m.groups) == 2 and m.groups[1].units == [1, 2] and m.unit_group == {0: 0, 1: 1, 2: 1}
    m.admit("a")
    m.ensure_capacity_batch({"a": 8})
    m.commit_lengths({"a": 8})
    # next query at position >= 8 sees keys >= 3: page 0 (keys 0..3) still holds key 3
    assert m.block_table(1, "a") == m.block_table(1, "a") and all(p >= 0 for p in m.block_table(1, "a"))
    m.ensure_capacity_batch({"a": 9})
    m.commit_lengths({"a": 9})  # keys >= 4 from now on: page 0 has passed
    windowed = m.block_table(1, "a")
    assert windowed[0] == -1 and all(p >= 0 for p in windowed[1:]) and len(windowed) == 3
    assert all(p >= 0 for p in m.block_table(0, "a"))  # the full group keeps everything
    for length in range(10, 40):
        m.ensure_capacity_batch({"a": length})
        m.commit_lengths({"a": length})
        held = [p for p in m.block_table(1, "a") if p >= 0]
        assert len(held) <= 3
        m.assert_invariants()
    assert m.groups[1].allocator.used_count <= 3 and m.groups[0].allocator.used_count == 10
    m.release("a")
    assert m.stats().pages_used == 0


def test_window_pool_is_sized_by_window_not_by_context():
    m = manager(unit_specs=[PagedKV(1, 8, window=8)], kv_tokens=4096, max_running=2, max_model_len=4096,
                prefill_chunk=16, page_size=4)
    assert m.groups[0].allocator.total_pages == 2 * (6 + 1)


def test_fixed_state_units_take_no_pages_and_disable_prefix_reuse():
    m = manager(unit_specs=[FixedState((4, 8)), PagedKV(2, 16)], prefix_cache_pages=8)
    assert m.state_units == {0: FixedState((4, 8))} and m.unit_group == {1: 0}
    assert m.prefix_cache_pages == 0
    only_state = manager(unit_specs=[FixedState((3,))])
    only_state.admit("a")
    only_state.ensure_capacity_batch({"a": 10})
    only_state.commit_lengths({"a": 10})
    assert only_state.length("a") == 10 and only_state.allocated_tokens("a") == 0


# -- prefix reuse ------------------------------------------------------------------------
def test_prefix_shared_by_different_tails_hits_and_last_token_is_never_covered():
    m = manager(prefix_cache_pages=8)
    first = list(range(10))
    assert m.admit("a", first) == 0 and m.prefix_cache_misses == 1
    m.ensure_capacity_batch({"a": 10})
    m.commit_lengths({"a": 10})
    pages = m.block_table(0, "a")
    m.release("a", first)
    stats = m.stats()
    assert (stats.request_pages_used, stats.prefix_pages_used, stats.pages_used) == (0, 2, 2)
    # same first 8 tokens, other tail: the two full pages are taken over, not copied
    assert m.admit("b", first[:8] + [77, 78, 79]) == 8 and m.block_table(0, "b") == pages[:2]
    assert m.length("b") == 8 and m.prefix_cache_hits == 1
    # a prompt that ends exactly on the page edge must still recompute its last token
    assert m.admit("c", first[:8]) == 4
    # a prompt that differs inside the first page misses
    assert m.admit("d", [9] + first[1:]) == 0
    m.assert_invariants()
    for rid in "bcd":
        m.release(rid)
    assert m.stats().pages_used == 2


def test_prefix_not_stored_on_preemption_nor_beyond_committed_length():
    m = manager(prefix_cache_pages=8)
    prompt = list(range(12))
    m.admit("a", prompt)
    m.ensure_capacity_batch({"a": 12})
    m.commit_lengths({"a": 6})  # only one full page computed so far
    m.release("a", prompt)
    assert m.stats().prefix_pages_used == 1
    m.admit("b", prompt)
    m.ensure_capacity_batch({"b": 12})
    m.commit_lengths({"b": 12})
    m.release("b")  # preempted: no prompt given
    assert m.stats().prefix_pages_used == 1


def test_prefix_published_by_a_live_request_is_shared_and_outlives_it():
    m = manager(prefix_cache_pages=8)
    prompt = list(range(10))
    m.admit("a", prompt)
    m.ensure_capacity_batch({"a": 10})
    m.commit_lengths({"a": 6})
    assert m.publish_prefix("a", prompt) == 4  # only what is committed
    m.commit_lengths({"a": 10})
    assert m.publish_prefix("a", prompt) == 8  # full pages before the last prompt token
    assert m.publish_prefix("a", prompt) == 8 and m.stats().prefix_pages_used == 2  # again: nothing new
    pages = m.block_table(0, "a")
    # a second request arrives while the first is still alive: same pages, three holders in all
    assert m.admit("b", prompt[:8] + [50, 51]) == 8 and m.block_table(0, "b") == pages[:2]
    assert set(m.groups[0].allocator.holders_of(pages[0])) == {"a", "b", PREFIX_HOLDER}
    m.ensure_capacity_batch({"a": 14, "b": 12})  # both go on writing behind the shared pages
    assert m.block_table(0, "a")[:2] == m.block_table(0, "b")[:2] and m.block_table(0, "a")[2] != m.block_table(0, "b")[2]
    m.assert_invariants()
    m.release("a")  # preempted or ended without storing: the index and b keep the pages
    assert m.groups[0].allocator.holders_of(pages[0]) == ("b", PREFIX_HOLDER) or \
        set(m.groups[0].allocator.holders_of(pages[0])) == {"b", PREFIX_HOLDER}
    m.release("b", prompt[:8] + [50, 51])
    assert m.stats().pages_used == 2 and m.publish_prefix("gone", prompt) == 0
    m.assert_invariants()


def test_prefix_entries_are_bounded_and_evicted_before_a_request_starves():
    m = manager(kv_tokens=32, prefix_cache_pages=3)  # 8 pages
    for i in range(3):
        prompt = [i] * 9
        m.admit(f"r{i}", prompt)
        m.ensure_capacity_batch({f"r{i}": 9})
        m.commit_lengths({f"r{i}": 9})
        m.release(f"r{i}", prompt)
    assert m.stats().prefix_pages_used == 3  # 6 wanted, bound 3
    m.admit("big")
    m.ensure_capacity_batch({"big": 32})  # needs all 8 pages: the index gives way
    assert m.stats().prefix_pages_used == 0 and m.stats().request_pages_used == 8
    m.assert_invariants()


def test_shared_pages_survive_index_pressure():
    m = manager(kv_tokens=32, prefix_cache_pages=4)
    prompt = list(range(9))
    m.admit("a", prompt)
    m.ensure_capacity_batch({"a": 9})
    m.commit_lengths({"a": 9})
    m.release("a", prompt)
    assert m.admit("b", prompt) == 8
    m.admit("c")
    with pytest.raises(CacheCapacityFull):
        m.ensure_capacity_batch({"c": 28})  # 7 pages, 6 free: b's shared pages cannot be evicted
    assert m.block_table(0, "b")[0] in [p for p in range(8) if PREFIX_HOLDER in m.groups[0].allocator.holders_of(p)]
    m.assert_invariants()


# -- what a paged need stores, byte statistics, room in the pool ---------------------------
def test_a_paged_need_says_what_it_stores():
    assert PagedKV(2, 16).numbers_per_token == 2 * (16 + 16) and PagedKV(2, 16).value_width == 16
    keys_only = PagedKV(1, 24, values=False)
    assert keys_only.value_width == 0 and keys_only.numbers_per_token == 24
    assert PagedKV(4, 8, value_dim=20).numbers_per_token == 4 * 28
    assert PagedKV(2, 16) != PagedKV(2, 16, value_dim=8), "another width is another group"
    with pytest.raises(ValueError):
        PagedKV(2, 16, values=False, value_dim=8)
    with pytest.raises(ValueError):
        PagedKV(0, 16)
    m = manager(unit_specs=[PagedKV(2, 16), PagedKV(2, 16, values=False), PagedKV(2, 16)])
    assert [g.units for g in m.groups] == [[0, 2], [1]]


def test_byte_statistics_follow_pages_and_tokens():
    """The reference's figures (src/cloud_engine/cache.py:503-526): reserved = used pages x page bytes over
    all layers, occupied = tokens x token bytes, the difference is lost inside pages that are not full."""
    m = manager(unit_specs=[PagedKV(2, 16)] * 3, element_bytes=2, prefix_cache_pages=8)  # pages of 4 tokens
    token_bytes = 2 * (16 + 16) * 2 * 3
    assert m.stats().reserved_bytes == m.stats().occupied_bytes == 0
    prompt = list(range(9))
    m.admit("a", prompt)
    m.ensure_capacity_batch({"a": 9})
    stats = m.stats()
    assert stats.reserved_bytes == 3 * 4 * token_bytes and stats.occupied_bytes == 0  # reserved before the step ran
    m.commit_lengths({"a": 9})
    stats = m.stats()
    assert stats.occupied_bytes == 9 * token_bytes
    assert stats.internal_fragmentation_bytes == 3 * token_bytes == stats.groups[0].internal_fragmentation_bytes
    # a page that the index and two requests share is counted once
    m.publish_prefix("a", prompt)
    assert m.admit("b", prompt[:8] + [70]) == 8
    m.ensure_capacity_batch({"b": 9})
    m.commit_lengths({"b": 9})
    stats = m.stats()
    assert stats.pages_used == 4 and stats.reserved_bytes == 16 * token_bytes and stats.occupied_bytes == 10 * token_bytes
    m.release("a", prompt), m.release("b")
    stats = m.stats()
    assert stats.reserved_bytes == stats.occupied_bytes == 8 * token_bytes  # the two indexed pages are full ones
    # groups report their own: a keys-only group of one unit in float32 beside keys and values
    two = manager(unit_specs=[PagedKV(2, 16), PagedKV(1, 8, values=False)], element_bytes=4)
    two.admit("x")
    two.ensure_capacity_batch({"x": 5})
    two.commit_lengths({"x": 5})
    first, second = two.stats().groups
    assert (first.reserved_bytes, first.occupied_bytes) == (8 * 64 * 4, 5 * 64 * 4)
    assert (second.reserved_bytes, second.occupied_bytes) == (8 * 8 * 4, 5 * 8 * 4)
    assert two.stats().internal_fragmentation_bytes == 3 * (64 + 8) * 4


def test_free_tokens_count_what_the_index_would_give_back():
    m = manager(kv_tokens=32, prefix_cache_pages=8)  # 8 pages of 4
    assert m.free_tokens() == 32
    prompt = list(range(13))
    m.admit("a", prompt)
    m.ensure_capacity_batch({"a": 13})
    m.commit_lengths({"a": 13})
    assert m.free_tokens() == 16
    m.release("a", prompt)  # three full pages stay in the index
    assert m.groups[0].allocator.free_count == 5 and m.free_tokens() == 32
    assert m.admit("b", prompt[:8] + [99]) == 8  # two of them are shared now: only the third can be evicted
    assert m.free_tokens() == 24
    m.ensure_capacity_batch({"b": 9 + 20})  # 6 more pages: 5 free and the evicted one
    assert m.free_tokens() == 0 and m.stats().prefix_pages_used == 2
    m.assert_invariants()
    only_state = manager(unit_specs=[FixedState((3,))])
    assert only_state.free_tokens() > 1 << 40, "a cache without pages never limits admission"


def test_a_copy_of_indexed_tokens_is_not_stored_below_the_page_the_index_has():
    """Two requests with the same first tokens are admitted before either has stored anything: each computes
    pages of its own.  The one that publishes second finds its tokens in the index on the other's pages; what it
    has below them must not be hung under those pages, which it does not hold: they would then be held by the index
    alone and yet not be evictable while it lives (two such pages once left a lone request without the one page
    it still needed, in a pool that had room for it)."""
    m = manager(kv_tokens=40, prefix_cache_pages=8)  # pages of 4 tokens, 10 pages
    common = list(range(8))
    first, second = common + [90, 91, 92], common + [70, 71, 72, 73, 74, 75]
    assert m.admit("first", first) == 0 and m.admit("second", second) == 0
    m.ensure_capacity_batch({"first": 11, "second": 14})
    m.commit_lengths({"first": 11, "second": 14})
    assert m.publish_prefix("first", first) == 8       # two pages of common tokens
    assert m.publish_prefix("second", second) == 0     # the same tokens on pages of its own: nothing stored under them
    m.assert_invariants()
    m.release("first", first)
    # what the index holds alone can be evicted, and free_tokens counts no more than that
    assert m.stats().prefix_pages_used == 2 and m.free_tokens() == (10 - 4) * 4
    m.ensure_capacity_batch({"second": 14 + 6 * 4})    # the second one grows into everything that is left
    assert m.stats().prefix_pages_used == 0
    m.assert_invariants()
    m.release("second", second)
    assert m.stats().pages_used == m.stats().prefix_pages_used == 3  # its own three full prompt pages, stored at its end
    m.clear_prefix_index()
    assert m.stats().pages_used == 0


def test_a_unit_of_several_needs_is_kept_cell_by_cell():
    """A mixer may need several things at once (``cache_need`` a tuple): pages and a state beside them, or two
    states.  Each is a cell; cells with equal paged needs share a group whichever unit they belong to."""
    from cie_amd.cache.manager import CacheManager, FixedState, PagedKV

    keys = PagedKV(2, 16)
    manager = CacheManager([keys, (keys, FixedState((3,), "int32")), None, (FixedState((2, 8)), FixedState((1,)))],
                           page_size=4, kv_tokens=32, max_running=2, max_model_len=16)
    assert manager.unit_cells == [0, (1, 2), 3, (4, 5)]
    assert manager.unit_group == {0: 0, 1: 0} and manager.groups[0].units == [0, 1]
    assert set(manager.state_units) == {2, 4, 5} and manager.unit_specs[3] is None
    manager.admit("a")
    manager.ensure_capacity_batch({"a": 9})
    manager.commit_lengths({"a": 9})
    assert manager.allocated_tokens("a") == 12 and manager.tokens_missing("a", 13) == 4
    manager.release("a")
    manager.assert_invariants()


def test_pool_size_from_free_memory_keeps_a_reserve():
    """Where no pool size is given the cache takes a share of the device memory that is free after the weights,
    less what a running engine needs beside it: the library's workspace and timing copies, a full step's
    activations and logits."""
    from cie_amd.cache.manager import FixedState, PagedKV
    from cie_amd.config import build_engine_config
    from cie_amd.engine.runner import reserve_bytes, tokens_from_bytes

    needs = [PagedKV(2, 128)] * 4 + [(PagedKV(2, 128), FixedState((8,)))]
    per_token = 5 * 2 * 256 * 2
    config = build_engine_config(max_model_len=1 << 15, max_running=1024, token_budget=2048, page_size=16,
                                 prefix_cache_pages=0)
    reserve = reserve_bytes(config, hidden_size=2048, vocab_size=150_000)
    assert reserve >= (64 << 20) + (640 << 20) + 2048 * 2048 * 64 + 2 * 1024 * 150_000 * 4
    free = 8 << 30
    tokens = tokens_from_bytes(config, needs, 2, free, 2048, 150_000)
    assert tokens == int((free - reserve) * 0.9) // per_token // 16 * 16
    assert reserve_bytes(build_engine_config(search_library_algorithms=False), 2048, 150_000) < reserve - (600 << 20)
    # less free memory than the reserve: one page, not a negative pool
    assert tokens_from_bytes(config, needs, 2, reserve // 2, 2048, 150_000) == 16
    # bytes given: taken as they are; never more than every slot full can use
    given = build_engine_config(base=config, kv_cache_bytes=per_token * 1000)
    assert tokens_from_bytes(given, needs, 2, 0, 2048, 150_000) == 992
    small = build_engine_config(max_model_len=64, max_running=2, page_size=16, prefix_cache_pages=3)
    assert tokens_from_bytes(small, needs, 2, free, 2048, 150_000) == (2 * 4 + 3) * 16
    assert tokens_from_bytes(config, [FixedState((4,))], 2, free, 64, 100) == 16  # nothing is paged
