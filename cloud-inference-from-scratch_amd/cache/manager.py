"""Host-side cache manager: pages, block tables, request slots, prefix reuse.

What the reference's ``PagedKVCache`` does on the host
(src/cloud_engine/cache.py:235-529) without its tensors: requests are admitted
with empty tables, a step's growth is all-or-nothing
(``ensure_capacity_batch``, cache.py:371-396), lengths advance only on commit
(cache.py:427-431), release gives every page back (cache.py:497-501).

Beyond the reference:

* The cache is a list of *units* (one per entry of the model's run order that
  writes a cache).  Units with the same need form a *group* with pages, an
  allocator and block tables of its own: ``PagedKV(window=None)`` keeps all
  keys, ``PagedKV(window=w)`` gives pages back once the window has passed them.
* A unit may hold several things at once (a mixer whose ``cache_need`` is a tuple: two states of different
  shape, or pages and a state beside them): each is a *cell* with a number of its own, and everything below
  (groups, states, the device side) is kept per cell; ``unit_cells`` says which cells a unit has.
* ``FixedState`` units get no pages; every request owns one *slot* (a row index
  below ``max_running``) from admission to release, which addresses both the
  fixed-size state rows and the request's row of the device block tables.
* Prefix reuse works on chained per-page keys and shares pages instead of
  copying them: the longest run of full prompt pages that an earlier request
  left is taken over read-only.  The reference keys whole aligned prompts and
  copies (cache.py:298-357).  The last prompt token is never covered, entries
  are bounded by ``prefix_cache_pages`` and evicted LRU before any request has
  to be preempted (cache.py:380).  It is active when the model has exactly one
  group and that group keeps all keys.
"""

from __future__ import annotations

from collections import OrderedDict
from collections.abc import Mapping, Sequence
from dataclasses import dataclass

from .allocator import CacheCapacityFull, PageAllocator

PREFIX_HOLDER = "\0prefix-index"


UNBOUNDED_TOKENS = 1 << 62   # what a cache without pages reports as free


@dataclass(frozen=True)
class PagedKV:
    """A mixer that appends per token, for each of ``kv_heads`` heads, a key of
    ``head_dim`` numbers and, if ``values``, a value of ``value_dim`` numbers
    (``None``: as wide as the key).  ``values=False`` is a cache of one vector
    per token and head (a latent that keys and values are both made from, or
    keys alone).  With a ``window`` only that many latest tokens are read."""

    kv_heads: int
    head_dim: int
    window: int | None = None
    values: bool = True
    value_dim: int | None = None

    def __post_init__(self) -> None:
        if self.kv_heads < 1 or self.head_dim < 1:
            raise ValueError("a paged cache needs at least one head of at least one number")
        if self.value_dim is not None and (not self.values or self.value_dim < 1):
            raise ValueError("value_dim needs values=True and a positive width")

    @property
    def value_width(self) -> int:
        """Numbers per value vector; 0 where none are stored."""
        if not self.values:
            return 0
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def numbers_per_token(self) -> int:
        return self.kv_heads * (self.head_dim + self.value_width)


@dataclass(frozen=True)
class FixedState:
    """A mixer that keeps a state of fixed ``shape`` per request."""

    shape: tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class GroupBytes:
    """One group's memory, as the reference's cache reports it for its single pool
    (src/cloud_engine/cache.py:503-526): ``reserved`` is what the used pages take in
    all the group's units, ``occupied`` what the tokens in them take, the rest is
    lost inside pages that are not full."""

    units: int
    pages_total: int
    pages_used: int
    reserved_bytes: int
    occupied_bytes: int

    @property
    def internal_fragmentation_bytes(self) -> int:
        return self.reserved_bytes - self.occupied_bytes


@dataclass(frozen=True)
class CacheStats:
    pages_total: int
    pages_used: int
    request_pages_used: int
    prefix_pages_used: int
    prefix_cache_hits: int
    prefix_cache_misses: int
    slots_used: int
    groups: tuple[GroupBytes, ...] = ()

    @property
    def utilization(self) -> float:
        return self.pages_used / self.pages_total if self.pages_total else 0.0

    @property
    def reserved_bytes(self) -> int:
        return sum(group.reserved_bytes for group in self.groups)

    @property
    def occupied_bytes(self) -> int:
        return sum(group.occupied_bytes for group in self.groups)

    @property
    def internal_fragmentation_bytes(self) -> int:
        return self.reserved_bytes - self.occupied_bytes


class _Group:
    def __init__(self, spec: PagedKV, units: list[int], num_pages: int, page_size: int,
                 most_per_request: int | None = None) -> None:
        self.spec = spec
        self.units = units
        self.most_per_request = most_per_request  # pages a request ever holds at once (a window group); None: no bound
        self.allocator = PageAllocator(num_pages, page_size)
        self.tables: dict[str, list[int]] = {}  # logical page index -> physical page, -1 once released


class _PrefixNode:
    __slots__ = ("key", "parent", "page", "children", "serial")
    _count = 0

    def __init__(self, key: tuple, parent: "_PrefixNode | None", page: int) -> None:
        self.key = key
        self.parent = parent
        self.page = page
        self.children = 0
        _PrefixNode._count += 1
        self.serial = _PrefixNode._count  # never reused, unlike id()


class CacheManager:
    def __init__(
        self,
        unit_specs: Sequence[PagedKV | FixedState | None],
        page_size: int,
        kv_tokens: int,
        max_running: int,
        max_model_len: int,
        prefill_chunk: int = 256,
        prefix_cache_pages: int = 0,
        element_bytes: int = 2,
    ) -> None:
        if page_size < 1 or page_size & (page_size - 1):
            raise ValueError(f"page_size must be a power of two, got {page_size}")
        if max_running < 1:
            raise ValueError("max_running must be positive")
        self.page_size = page_size
        self.max_running = max_running
        self.max_model_len = max_model_len
        self.element_bytes = element_bytes  # of one cached number; only the byte statistics use it
        self.table_width = -(-max_model_len // page_size)
        # a unit's need may be a tuple of needs: every need becomes a cell; a unit with one need is its own cell
        cells: list[PagedKV | FixedState | None] = []
        self.unit_cells: list[int | tuple[int, ...]] = []
        for spec in unit_specs:
            if isinstance(spec, (tuple, list)):
                self.unit_cells.append(tuple(range(len(cells), len(cells) + len(spec))))
                cells.extend(spec)
            else:
                self.unit_cells.append(len(cells))
                cells.append(spec)
        self.unit_specs = tuple(cells)
        self.groups: list[_Group] = []
        self.unit_group: dict[int, int] = {}
        self.state_units: dict[int, FixedState] = {}
        by_spec: dict[PagedKV, int] = {}
        full_pages = kv_tokens // page_size
        if full_pages < 1:
            raise ValueError("kv_tokens too small for even one page")
        for unit, spec in enumerate(self.unit_specs):
            if isinstance(spec, PagedKV):
                if spec not in by_spec:
                    pages, per_request = full_pages, None
                    if spec.window is not None:
                        per_request = -(-(spec.window + prefill_chunk) // page_size) + 1
                        pages = min(full_pages, max_running * per_request)
                    by_spec[spec] = len(self.groups)
                    self.groups.append(_Group(spec, [], pages, page_size, per_request))
                index = by_spec[spec]
                self.groups[index].units.append(unit)
                self.unit_group[unit] = index
            elif isinstance(spec, FixedState):
                self.state_units[unit] = spec
            elif spec is not None:
                raise TypeError(f"cache unit {unit}: unknown need {spec!r}")
        self._free_slots = list(range(max_running - 1, -1, -1))
        self._slots: dict[str, int] = {}
        self._length: dict[str, int] = {}
        self._dirty: set[tuple[int, int]] = set()  # (group, slot) rows the device copy lacks
        self._slot_serial: dict[int, int] = {}
        self._fresh_slots: set[int] = set()  # slots whose fixed state must be cleared before use
        self.prefix_cache_pages = (
            prefix_cache_pages
            if len(self.groups) == 1 and self.groups[0].spec.window is None and not self.state_units
            else 0
        )
        self._prefix: OrderedDict[tuple, _PrefixNode] = OrderedDict()  # LRU order, oldest first
        self.prefix_cache_hits = 0
        self.prefix_cache_misses = 0

    # -- queries --------------------------------------------------------------
    def slot(self, request_id: str) -> int:
        return self._slots[request_id]

    def length(self, request_id: str) -> int:
        return self._length[request_id]

    def has(self, request_id: str) -> bool:
        return request_id in self._slots

    def block_table(self, group: int, request_id: str) -> list[int]:
        return list(self.groups[group].tables[request_id])

    def allocated_tokens(self, request_id: str) -> int:
        if request_id not in self._slots:
            return 0
        held = max((sum(1 for p in g.tables[request_id] if p >= 0) for g in self.groups), default=0)
        return held * self.page_size

    def free_tokens(self) -> int:
        """Tokens the pool could take now: the free pages of the scarcest group, and with them the
        pages that only the prefix index holds, which growth evicts when it needs them.  A cache
        without pages (every unit a fixed state, or none) is never the limit."""
        if not self.groups:
            return UNBOUNDED_TOKENS
        pages = []
        for index, group in enumerate(self.groups):
            free = group.allocator.free_count
            if index == 0 and self._prefix:
                # a page that a request shares keeps its ancestors shared too, so every page held by
                # the index alone can be evicted, leaves first
                free += sum(1 for node in self._prefix.values()
                            if group.allocator.holders_of(node.page) == (PREFIX_HOLDER,))
            pages.append(free)
        return min(pages) * self.page_size

    def tokens_missing(self, request_id: str, upto: int) -> int:
        """What ``request_id`` (admitted or not) would still take of :meth:`free_tokens` to hold ``upto``
        tokens: the pages it lacks in the group where it lacks most, times the page size.  A group that
        keeps a window never holds more than the window and one step's portion."""
        most = 0
        for group in self.groups:
            pages = group.allocator.pages_for(upto)
            if group.most_per_request is not None:
                pages = min(pages, group.most_per_request)
            table = group.tables.get(request_id, ())
            most = max(most, pages - sum(1 for page in table if page >= 0))
        return max(0, most) * self.page_size

    def take_dirty_rows(self) -> list[tuple[int, int, list[int]]]:
        """(group, slot, table) of every block-table row that changed since the last call."""
        by_slot = {slot: rid for rid, slot in self._slots.items()}
        rows = []
        for group, slot in sorted(self._dirty):
            rid = by_slot.get(slot)
            rows.append((group, slot, list(self.groups[group].tables[rid]) if rid is not None else []))
        self._dirty.clear()
        return rows

    def slot_serial(self, slot: int) -> int:
        """How many requests have been given this slot so far: tells the device side whether a dirty
        row still belongs to the request whose table it has already copied."""
        return self._slot_serial.get(slot, 0)

    def take_fresh_slots(self) -> list[int]:
        fresh = sorted(self._fresh_slots)
        self._fresh_slots.clear()
        return fresh

    # -- admission ------------------------------------------------------------
    def admit(self, request_id: str, prompt_tokens: Sequence[int] | None = None) -> int:
        """Give the request a slot and empty tables; returns how many leading
        prompt tokens are already cached (taken over from the prefix index)."""
        if request_id in self._slots:
            raise ValueError(f"duplicate admission of {request_id}")
        if request_id == PREFIX_HOLDER:
            raise ValueError("reserved request id")
        if not self._free_slots:
            raise CacheCapacityFull(f"all {self.max_running} request slots are taken")
        slot = self._free_slots.pop()
        self._slots[request_id] = slot
        self._slot_serial[slot] = self._slot_serial.get(slot, 0) + 1
        self._length[request_id] = 0
        self._fresh_slots.add(slot)
        for index, group in enumerate(self.groups):
            group.tables[request_id] = []
            self._dirty.add((index, slot))
        if prompt_tokens is not None and self.prefix_cache_pages:
            return self._restore_prefix(request_id, prompt_tokens)
        return 0

    # -- growth ---------------------------------------------------------------
    def _missing(self, group: _Group, request_id: str, tokens: int) -> int:
        return max(0, group.allocator.pages_for(tokens) - len(group.tables[request_id]))

    def ensure_capacity_batch(self, required_tokens: Mapping[str, int]) -> None:
        """Grow every named request's tables to hold ``required_tokens[id]``
        tokens, in every group, or change nothing and raise CacheCapacityFull."""
        for request_id, tokens in required_tokens.items():
            if request_id not in self._slots:
                raise KeyError(f"request {request_id!r} has no block table")
            if tokens > self.max_model_len:
                raise ValueError(f"{tokens} tokens exceed max_model_len {self.max_model_len}")
        additions = []
        for group in self.groups:
            extra = {rid: self._missing(group, rid, tokens) for rid, tokens in required_tokens.items()}
            total = sum(extra.values())
            if total > group.allocator.free_count and self.prefix_cache_pages:
                self._evict_prefix_pages(total)
            if not group.allocator.can_satisfy(total):
                raise CacheCapacityFull(
                    f"need {total} additional pages, {group.allocator.free_count} free"
                )
            additions.append(extra)
        for index, (group, extra) in enumerate(zip(self.groups, additions)):
            for request_id, count in extra.items():
                if count:
                    group.tables[request_id].extend(group.allocator.allocate(request_id, count))
                    self._dirty.add((index, self._slots[request_id]))

    def commit_lengths(self, lengths: Mapping[str, int]) -> None:
        """The step succeeded: advance lengths, give back pages a window has passed."""
        for request_id, length in lengths.items():
            for group in self.groups:
                if group.allocator.pages_for(length) > len(group.tables[request_id]):
                    raise RuntimeError(f"length {length} exceeds allocated table for {request_id}")
            self._length[request_id] = max(self._length[request_id], length)
        for index, group in enumerate(self.groups):
            window = group.spec.window
            if window is None:
                continue
            for request_id in lengths:
                # the next query sits at position >= length and sees keys >= length + 1 - window
                first_needed = max(0, self._length[request_id] + 1 - window)
                table = group.tables[request_id]
                passed = [i for i in range(min(first_needed // self.page_size, len(table))) if table[i] >= 0]
                if passed:
                    group.allocator.free([table[i] for i in passed], request_id)
                    for i in passed:
                        table[i] = -1
                    self._dirty.add((index, self._slots[request_id]))

    # -- release --------------------------------------------------------------
    def release(self, request_id: str, prompt_tokens: Sequence[int] | None = None) -> None:
        """Give back the request's slot and pages.  With ``prompt_tokens`` its full
        prompt pages are first offered to the prefix index (not on preemption)."""
        if request_id not in self._slots:
            return
        if prompt_tokens is not None and self.prefix_cache_pages:
            self._store_prefix(request_id, prompt_tokens)
        slot = self._slots.pop(request_id)
        for index, group in enumerate(self.groups):
            table = group.tables.pop(request_id)
            held = [page for page in table if page >= 0]
            if held:
                group.allocator.free(held, request_id)
            self._dirty.add((index, slot))
        self._length.pop(request_id, None)
        self._free_slots.append(slot)

    # -- prefix index -----------------------------------------------------------
    def publish_prefix(self, request_id: str, prompt_tokens: Sequence[int]) -> int:
        """Offer the full prompt pages a live request has committed to the prefix index; the request
        keeps them (a page then has two holders and is read-only for both).  Returns the tokens indexed."""
        if request_id not in self._slots or not self.prefix_cache_pages:
            return 0
        return self._store_prefix(request_id, prompt_tokens)

    def _restore_prefix(self, request_id: str, tokens: Sequence[int]) -> int:
        group = self.groups[0]
        candidate_pages = (len(tokens) - 1) // self.page_size
        matched: list[_PrefixNode] = []
        parent_id: int | None = None
        for i in range(candidate_pages):
            key = (parent_id, tuple(tokens[i * self.page_size:(i + 1) * self.page_size]))
            node = self._prefix.get(key)
            if node is None:
                break
            matched.append(node)
            parent_id = node.serial
        if not matched:
            if candidate_pages:
                self.prefix_cache_misses += 1
            return 0
        table = group.tables[request_id]
        for node in matched:
            group.allocator.retain(node.page, request_id)
            table.append(node.page)
            self._prefix.move_to_end(node.key)
        self._dirty.add((0, self._slots[request_id]))
        length = len(matched) * self.page_size
        self._length[request_id] = length
        self.prefix_cache_hits += 1
        return length

    def _store_prefix(self, request_id: str, tokens: Sequence[int]) -> int:
        group = self.groups[0]
        table = group.tables[request_id]
        pages = min((len(tokens) - 1) // self.page_size, self._length[request_id] // self.page_size, len(table))
        parent: _PrefixNode | None = None
        stored = 0
        for i in range(pages):
            key = (parent.serial if parent is not None else None,
                   tuple(tokens[i * self.page_size:(i + 1) * self.page_size]))
            node = self._prefix.get(key)
            if node is None:
                if len(self._prefix) >= self.prefix_cache_pages and not self._evict_one(protect=parent):
                    break
                node = _PrefixNode(key, parent, table[i])
                group.allocator.retain(table[i], PREFIX_HOLDER)
                self._prefix[key] = node
                if parent is not None:
                    parent.children += 1
            elif node.page != table[i]:
                # The index has these tokens on another page: a request that came after this one was admitted
                # stored them first, and this one computed a copy of its own.  What lies below is not stored
                # under that page: whoever holds a page of the index must hold all above it, or the pages
                # above could not be evicted while the request lives although only the index holds them.
                break
            else:
                self._prefix.move_to_end(key)
            parent = node
            stored += 1
        return stored * self.page_size

    def _evict_one(self, protect: _PrefixNode | None = None) -> bool:
        """Drop the least recently used leaf of the index that no request shares
        (a shared page stays indexed: the index is what marks it read-only)."""
        group = self.groups[0]
        ancestors = set()
        node = protect
        while node is not None:
            ancestors.add(node.serial)
            node = node.parent
        for key, node in self._prefix.items():
            if node.children or node.serial in ancestors:
                continue
            if group.allocator.holders_of(node.page) != (PREFIX_HOLDER,):
                continue
            del self._prefix[key]
            if node.parent is not None:
                node.parent.children -= 1
            group.allocator.free([node.page], PREFIX_HOLDER)
            return True
        return False

    def _evict_prefix_pages(self, needed: int) -> None:
        group = self.groups[0]
        while group.allocator.free_count < needed and self._evict_one():
            pass

    def clear_prefix_index(self) -> None:
        while self._evict_one():
            pass

    # -- accounting -------------------------------------------------------------
    def _group_bytes(self, index: int, group: _Group) -> GroupBytes:
        """Tokens are counted once per page, however many hold it; a shared page is a full one."""
        size = self.page_size
        filled: dict[int, int] = {}
        for request_id, table in group.tables.items():
            length = self._length.get(request_id, 0)
            for place, page in enumerate(table):
                if page >= 0:
                    filled[page] = max(filled.get(page, 0), min(size, max(0, length - place * size)))
        if index == 0:
            for node in self._prefix.values():
                filled[node.page] = size
        token_bytes = group.spec.numbers_per_token * self.element_bytes * len(group.units)
        used = group.allocator.used_count
        return GroupBytes(units=len(group.units), pages_total=group.allocator.total_pages, pages_used=used,
                          reserved_bytes=used * size * token_bytes,
                          occupied_bytes=sum(filled.values()) * token_bytes)

    def stats(self) -> CacheStats:
        request_pages = 0
        for group in self.groups:
            allocator = group.allocator
            request_pages += sum(1 for page in list(allocator._holders)
                                 if any(holder != PREFIX_HOLDER for holder in allocator.holders_of(page)))
        return CacheStats(
            pages_total=sum(g.allocator.total_pages for g in self.groups),
            pages_used=sum(g.allocator.used_count for g in self.groups),
            request_pages_used=request_pages,
            prefix_pages_used=len(self._prefix),
            prefix_cache_hits=self.prefix_cache_hits,
            prefix_cache_misses=self.prefix_cache_misses,
            slots_used=len(self._slots),
            groups=tuple(self._group_bytes(i, g) for i, g in enumerate(self.groups)),
        )

    def assert_invariants(self) -> None:
        for group in self.groups:
            group.allocator.assert_invariants()
            writers: dict[int, str] = {}
            for request_id, table in group.tables.items():
                live = [page for page in table if page >= 0]
                assert len(set(live)) == len(live), f"{request_id} lists a page twice"
                for page in live:
                    holders = group.allocator.holders_of(page)
                    assert request_id in holders, f"{request_id} lists page {page} it does not hold"
                    if PREFIX_HOLDER not in holders:
                        assert page not in writers, f"page {page} held by {writers[page]} and {request_id}"
                        writers[page] = request_id
            listed = {page for table in group.tables.values() for page in table if page >= 0}
            indexed = {node.page for node in self._prefix.values()} if group is self.groups[0] else set()
            assert listed | indexed == set(group.allocator._holders), "a used page is in no table"
        if self.groups:
            holders_of = self.groups[0].allocator.holders_of
            for node in self._prefix.values():
                if node.parent is not None:
                    missing = set(holders_of(node.page)) - set(holders_of(node.parent.page))
                    assert not missing, f"{sorted(missing)} hold page {node.page} of the index but not the page above it"
        assert len(self._slots) + len(self._free_slots) == self.max_running, "request slot lost"
        assert len(set(self._slots.values())) == len(self._slots), "two requests share a slot"
