"""The cache manager: who holds which pages and which state slot.

Cache entries (one per mixer execution that keeps something between steps) are sorted
into *groups*. Entries with equal paged needs (kv heads, head size, retention rule) form
one page group with a pool of its own and one block table per request; a page id
addresses the same page in every entry of the group. Entries with fixed-size state share
the request's *slot*: one index into every state tensor. Slots exist even when the model
has no such state.

Lifetime of a request: ``admit`` (takes a slot, zeroes its state) -> per step ``reserve``
(maps pages for the tokens the step will append; all or nothing) and ``commit`` (the new
length; a windowed group gives back the pages its window has passed) -> ``release``
(everything back to the pools). The reference reserves one contiguous arena per slot for
the whole context instead (native/src/v2_runtime.cpp:20700-20758) and zeroes it on reset
(:20437-20451).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch

from .needs import FixedState, PagedKV
from .pages import CacheAccountingError, OutOfPages, PagePool, SlotPool

NO_PAGE = -1


@dataclass
class PageGroup:
    key: Tuple
    need: PagedKV
    entries: List[int]
    pool: PagePool
    tables: Dict[Hashable, List[int]] = field(default_factory=dict)   # request -> page per block (NO_PAGE if given back)


@dataclass
class _Request:
    slot: int
    length: int = 0


class CacheManager:
    def __init__(self, needs: Mapping[int, object], num_pages: int, max_requests: int, page_size: int = 64,
                 max_pages_per_request: Optional[int] = None, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None):
        """``needs``: cache entry id -> PagedKV | FixedState. ``num_pages``: pages of every
        page group. ``device`` None keeps the bookkeeping only (no storage)."""
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_requests = max_requests
        self.max_pages_per_request = max_pages_per_request or num_pages
        self.dtype = dtype
        self.device = device
        self.groups: List[PageGroup] = []
        self.entry_group: Dict[int, int] = {}
        self.state_entries: Dict[int, FixedState] = {}
        by_key: Dict[Tuple, PageGroup] = {}
        for entry in sorted(needs):
            need = needs[entry]
            if isinstance(need, PagedKV):
                group = by_key.get(need.group_key())
                if group is None:
                    group = PageGroup(need.group_key(), need, [], PagePool(num_pages))
                    by_key[need.group_key()] = group
                    self.groups.append(group)
                group.entries.append(entry)
                self.entry_group[entry] = self.groups.index(group)
            elif isinstance(need, FixedState):
                self.state_entries[entry] = need
            elif need is not None:
                raise TypeError(f"cache entry {entry}: unknown need {need!r}")
        self.slots = SlotPool(max_requests)
        self.requests: Dict[Hashable, _Request] = {}
        # storage
        self.k_pages: Dict[int, torch.Tensor] = {}
        self.v_pages: Dict[int, torch.Tensor] = {}
        self.state: Dict[int, torch.Tensor] = {}
        if device is not None:
            for group in self.groups:
                n = group.need
                for entry in group.entries:
                    # K keeps a key's channels together, V a channel's tokens (see the attention kernels)
                    self.k_pages[entry] = torch.zeros((num_pages, n.num_kv_heads, page_size, n.head_dim), dtype=dtype, device=device)
                    self.v_pages[entry] = torch.zeros((num_pages, n.num_kv_heads, n.head_dim, page_size), dtype=dtype, device=device)
            for entry, need in self.state_entries.items():
                self.state[entry] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    # ----- sizes ------------------------------------------------------------------------
    def pages_for(self, tokens: int) -> int:
        return (tokens + self.page_size - 1) // self.page_size

    def _first_needed_block(self, group: PageGroup, length: int) -> int:
        """Blocks before this one hold only keys the window has passed once the sequence
        is ``length`` tokens long (the next query sits at position ``length``)."""
        if group.need.window is None:
            return 0
        first_key = max(0, length - group.need.window + 1)
        return first_key // self.page_size

    def pages_missing(self, request: Hashable, new_length: int) -> Dict[int, int]:
        """Per group: pages a reservation up to ``new_length`` would have to take."""
        missing = {}
        blocks = self.pages_for(new_length)
        for index, group in enumerate(self.groups):
            table = group.tables.get(request, [])
            missing[index] = max(0, blocks - len(table))
        return missing

    def can_reserve(self, request: Hashable, new_length: int, spare: int = 0) -> bool:
        if self.pages_for(new_length) > self.max_pages_per_request:
            return False
        return all(self.groups[g].pool.free_count - spare >= n for g, n in self.pages_missing(request, new_length).items())

    def free_pages(self) -> int:
        """Free pages of the tightest group (all groups, if there are none: unlimited)."""
        return min((g.pool.free_count for g in self.groups), default=1 << 30)

    # ----- lifetime ---------------------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        if request in self.requests:
            raise CacheAccountingError(f"request {request!r} is already live")
        slot = self.slots.alloc()
        self.requests[request] = _Request(slot)
        for group in self.groups:
            group.tables[request] = []
        for tensor in self.state.values():
            tensor[slot].zero_()
        return slot

    def slot_of(self, request: Hashable) -> int:
        return self.requests[request].slot

    def length_of(self, request: Hashable) -> int:
        return self.requests[request].length

    def reserve(self, request: Hashable, new_length: int) -> None:
        """Map pages for positions < new_length in every group, or raise OutOfPages and
        change nothing."""
        if request not in self.requests:
            raise KeyError(f"request {request!r} is not live")
        if self.pages_for(new_length) > self.max_pages_per_request:
            raise OutOfPages(f"request {request!r} would need {self.pages_for(new_length)} pages; "
                             f"a block table holds {self.max_pages_per_request}")
        missing = self.pages_missing(request, new_length)
        for g, count in missing.items():
            if self.groups[g].pool.free_count < count:
                raise OutOfPages(f"out of cache pages: request {request!r} needs {count} more, "
                                 f"{self.groups[g].pool.free_count} free")
        for g, count in missing.items():
            group = self.groups[g]
            table = group.tables[request]
            for _ in range(count):
                table.append(group.pool.alloc())

    def commit(self, request: Hashable, new_length: int) -> None:
        state = self.requests[request]
        if new_length < state.length:
            raise ValueError("a sequence does not shrink")
        state.length = new_length
        for group in self.groups:
            table = group.tables[request]
            for block in range(min(self._first_needed_block(group, new_length), len(table))):
                if table[block] != NO_PAGE:
                    group.pool.free(table[block])
                    table[block] = NO_PAGE

    def release(self, request: Hashable) -> None:
        if request not in self.requests:
            raise CacheAccountingError(f"request {request!r} is released but not live")
        state = self.requests.pop(request)
        for group in self.groups:
            for page in group.tables.pop(request):
                if page != NO_PAGE:
                    group.pool.free(page)
        self.slots.free(state.slot)

    # ----- views for the step function ---------------------------------------------------
    def block_table_rows(self, group_index: int, requests: Sequence[Hashable], stride: Optional[int] = None) -> np.ndarray:
        group = self.groups[group_index]
        stride = stride or max([len(group.tables[r]) for r in requests] + [1])
        rows = np.full((len(requests), stride), 0, dtype=np.int32)
        for i, request in enumerate(requests):
            table = group.tables[request]
            # a page that was given back is never read (the window has passed it); any valid id will do
            rows[i, :len(table)] = [p if p != NO_PAGE else 0 for p in table]
        return rows

    # ----- accounting -------------------------------------------------------------------
    def check_invariants(self) -> None:
        """No page lost, none held twice; slots likewise."""
        for group in self.groups:
            held = [p for table in group.tables.values() for p in table if p != NO_PAGE]
            if len(held) != len(set(held)):
                raise CacheAccountingError("a page is held by two block tables")
            if len(held) != group.pool.in_use:
                raise CacheAccountingError(f"{group.pool.in_use} pages are out of the pool but tables hold {len(held)}")
            if any(not group.pool.is_held(p) for p in held):
                raise CacheAccountingError("a block table holds a page the pool believes free")
            if set(group.tables) != set(self.requests):
                raise CacheAccountingError("block tables and live requests differ")
        slots = [r.slot for r in self.requests.values()]
        if len(slots) != len(set(slots)) or len(slots) != self.slots.num_slots - self.slots.free_count:
            raise CacheAccountingError("slot accounting is off")

    def stats(self) -> Dict[str, int]:
        return {
            "pages_total": self.num_pages,
            "pages_free": self.free_pages() if self.groups else self.num_pages,
            "pages_peak": max((g.pool.peak_in_use for g in self.groups), default=0),
            "slots_free": self.slots.free_count,
            "live_requests": len(self.requests),
        }
