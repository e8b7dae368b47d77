"""Device side of the cache: page pools, block tables and state rows.

For every group of the :class:`~cie_amd.cache.manager.CacheManager` a pool of
keys ``[units, pages, kv_heads, page_size, head_dim]`` and, where the group's
need stores values, a pool of values ``[units, pages, kv_heads, value_width,
page_size]``, transposed: the layouts the matrix-core attention reads with plain
vector loads, a page of one head contiguous.  (A need with ``values=False`` has
the key pool only; its mixer decides what the one vector per token means.)
Beside them one int32 block table ``[max_running, width]`` whose row ``slot``
holds the request's host table in its first entries.  The reference keeps ``[layers, pages, page_size, kv_heads, head_dim]``
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
        self.key_pools: list[torch.Tensor] = []
        self.value_pools: list[torch.Tensor | None] = []
        self.tables: list[torch.Tensor] = []
        self.pad_slot = manager.max_running
        self._row_seen: dict[tuple[int, int], tuple[int, int]] = {}  # (group, slot) -> (slot serial, entries copied)
        for group in manager.groups:
            spec = group.spec
            pad_page = group.allocator.total_pages
            units, pages, size = len(group.units), pad_page + 1, manager.page_size
            self.key_pools.append(torch.zeros((units, pages, spec.kv_heads, size, spec.head_dim),
                                              dtype=dtype, device=device))
            self.value_pools.append(torch.zeros((units, pages, spec.kv_heads, spec.value_width, size),
                                                dtype=dtype, device=device) if spec.values else None)
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
                values = self.value_pools[index]
                self._views[unit] = PagedView(self.key_pools[index][local],
                                              values[local] if values is not None else None,
                                              self.tables[index], manager.page_size)
            elif unit in self.states:
                self._views[unit] = StateView(self.states[unit])
            else:
                self._views[unit] = None

    def view(self, unit: int) -> Any:
        """What the mixer of cache unit ``unit`` is handed: a ``PagedView``, a ``StateView``, nothing, or,
        for a mixer whose need is a tuple, the tuple of its views in the same order."""
        cells = self.manager.unit_cells[unit]
        if isinstance(cells, tuple):
            return tuple(self._views[cell] for cell in cells)
        return self._views[cells]

    def bytes(self) -> int:
        pools = self.key_pools + [p for p in self.value_pools if p is not None]
        return sum(p.numel() * p.element_size() for p in pools)

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
