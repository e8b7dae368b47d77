"""Page allocator: a LIFO free list over fixed-size pages with named holders.

Same contract as the reference's ``BlockAllocator``
(src/cloud_engine/cache.py:80-155): ``free + used == total``, a failed call
changes nothing, freeing what one does not hold raises.  One extension: a live
page may get further holders through :meth:`retain` (a full prompt page shared
read-only by the prefix index and by requests); it returns to the free list
when its last holder lets go.  Pure Python, no torch.
"""

from __future__ import annotations

from collections.abc import Sequence


class CacheCapacityFull(Exception):
    """Not enough free pages (or request slots) for what a step needs."""

    is_capacity_error = True


class DoubleFreeError(ValueError):
    """A page was released by someone who does not hold it, or twice in one call."""


class PageAllocator:
    def __init__(self, num_pages: int, page_size: int) -> None:
        if num_pages < 1:
            raise ValueError("num_pages must be positive")
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.total_pages = num_pages
        self.page_size = page_size
        self._free: list[int] = list(range(num_pages - 1, -1, -1))  # pop() hands out 0, 1, 2, ...
        self._holders: dict[int, list[str]] = {}

    # -- accounting ---------------------------------------------------------
    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return len(self._holders)

    def pages_for(self, tokens: int) -> int:
        if tokens < 0:
            raise ValueError("tokens must be non-negative")
        return -(-tokens // self.page_size)

    def can_satisfy(self, n_pages: int) -> bool:
        return n_pages <= self.free_count

    def held_by(self, holder: str) -> int:
        return sum(holders.count(holder) for holders in self._holders.values())

    def holders_of(self, page: int) -> tuple[str, ...]:
        return tuple(self._holders.get(page, ()))

    # -- mutation -----------------------------------------------------------
    def allocate(self, holder: str, n_pages: int) -> list[int]:
        if n_pages < 0:
            raise ValueError("n_pages must be non-negative")
        if n_pages > self.free_count:
            raise CacheCapacityFull(f"requested {n_pages} pages, only {self.free_count} free")
        pages = [self._free.pop() for _ in range(n_pages)]
        for page in pages:
            self._holders[page] = [holder]
        return pages

    def retain(self, page: int, holder: str) -> None:
        """Add ``holder`` to a page that is already live."""
        holders = self._holders.get(page)
        if holders is None:
            raise DoubleFreeError(f"page {page} is free and cannot be retained by {holder!r}")
        if holder in holders:
            raise DoubleFreeError(f"page {page} is already held by {holder!r}")
        holders.append(holder)

    def free(self, pages: Sequence[int], holder: str) -> list[int]:
        """Drop ``holder`` from each page; returns the pages that became free.
        Raises before changing anything if any page is not held by ``holder``."""
        if len(set(pages)) != len(pages):
            raise DoubleFreeError("same page freed twice in one call")
        for page in pages:
            holders = self._holders.get(page)
            if holders is None:
                raise DoubleFreeError(f"page {page} is already free")
            if holder not in holders:
                raise DoubleFreeError(f"page {page} held by {holders!r}, freed by {holder!r}")
        returned = []
        for page in pages:
            holders = self._holders[page]
            holders.remove(holder)
            if not holders:
                del self._holders[page]
                self._free.append(page)
                returned.append(page)
        return returned

    def free_for(self, holder: str) -> list[int]:
        held = [page for page, holders in self._holders.items() if holder in holders]
        self.free(held, holder)
        return held

    def assert_invariants(self) -> None:
        assert len(self._holders) + len(self._free) == self.total_pages, "page lost: free + used != total"
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        assert not set(self._free) & set(self._holders), "a page is both free and held"
        assert all(0 <= page < self.total_pages for page in self._free)
        assert all(holders and len(set(holders)) == len(holders) for holders in self._holders.values())
