"""Device side of the cache: page pools, block tables and state rows.

For every group of the :class:`~cie_amd.cache.manager.CacheManager` one pool
``[units, 2, pages, kv_heads, page_size * head_dim]`` (keys at index 0 of the
second axis as ``[page_size, head_dim]``, values at index 1 transposed as
``[head_dim, page_size]``, the layouts the matrix-core attention reads with plain
vector loads; a page of one head is contiguous) and one int32 block
table ``[max_running, width]`` whose row ``slot`` holds the request's host
table in its first entries.  The reference keeps ``[layers, pages, page_size, kv_heads, head_dim]``
pools (src/cloud_engine/cache.py:266-274) and uploads padded tables every step
(src/cloud_engine/engine.py:264-278); here only rows that changed are copied.

One page and one slot beyond the manager's are kept for padding: a captured
decode graph runs a fixed number of rows, and the rows that no request fills
use slot ``pad_slot``, whose block table points at page ``pad_page`` only.
(The reference pads by repeating the last real row, which writes that row's
cache slot twice, src/cloud_engine/engine.py:329-356.)
"""

from __future__ import annotations

from typing import Any

import torch

from ..cache.manager import CacheManager, FixedState
from .batch import PagedView, StateView, to_device_staging

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class DeviceCache:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device: torch.device) -> None:
        self.manager = manager
        self.dtype = dtype
        self.device = device
        self.pools: list[torch.Tensor] = []
        self.tables: list[torch.Tensor] = []
        self.pad_slot = manager.max_running
        self._row_seen: dict[tuple[int, int], tuple[int, int]] = {}  # (group, slot) -> (slot serial, entries copied)
        for group in manager.groups:
            spec = group.spec
            pad_page = group.allocator.total_pages
            shape = (len(group.units), 2, pad_page + 1, spec.kv_heads, manager.page_size, spec.head_dim)
            self.pools.append(torch.zeros(shape, dtype=dtype, device=device))
            table = torch.zeros((manager.max_running + 1, manager.table_width), dtype=torch.int32, device=device)
            table[self.pad_slot] = pad_page
            self.tables.append(table)
        self.states: dict[int, torch.Tensor] = {}
        for unit, spec in manager.state_units.items():
            assert isinstance(spec, FixedState)
            self.states[unit] = torch.zeros((manager.max_running + 1, *spec.shape),
                                            dtype=_STATE_DTYPES[spec.dtype], device=device)
        self._views: dict[int, Any] = {}
        for unit in range(len(manager.unit_specs)):
            if unit in manager.unit_group:
                index = manager.unit_group[unit]
                local = manager.groups[index].units.index(unit)
                pool = self.pools[index]
                spec = manager.groups[index].spec
                pages = manager.groups[index].allocator.total_pages + 1
                values = pool[local, 1].view(pages, spec.kv_heads, spec.head_dim, manager.page_size)
                self._views[unit] = PagedView(pool[local, 0], values, self.tables[index], manager.page_size)
            elif unit in self.states:
                self._views[unit] = StateView(self.states[unit])
            else:
                self._views[unit] = None

    def view(self, unit: int) -> Any:
        return self._views[unit]

    def bytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.pools)

    def sync(self) -> None:
        """Bring the device block tables up to the host's; clear the state of
        slots that were handed to a new request."""
        for group, slot, table in self.manager.take_dirty_rows():
            # A request's table only grows at its end (pages a window has passed turn to -1 in place, and
            # are never read again): copy what was appended since the last time, all of it once the slot
            # has gone to another request.  Entries past the request's pages keep what they held; nothing
            # reads them.
            serial = self.manager.slot_serial(slot)
            seen, synced = self._row_seen.get((group, slot), (-1, 0))
            first = synced if seen == serial and synced <= len(table) else 0
            if len(table) > first:
                staged = to_device_staging([max(p, 0) for p in table[first:]], self.device)
                self.tables[group][slot, first: len(table)].copy_(staged, non_blocking=True)
            self._row_seen[(group, slot)] = (serial, len(table))
        fresh = self.manager.take_fresh_slots()
        if fresh and self.states:
            for state in self.states.values():
                state[fresh] = 0
