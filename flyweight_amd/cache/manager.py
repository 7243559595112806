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
(everything back to the pools). The bookkeeping is the host library's (C++,
``csrc/host/cache.hpp``); this class is its Python face and owns the tensors. The reference reserves one contiguous arena per slot for
the whole context instead (native/src/v2_runtime.cpp:20700-20758) and zeroes it on reset
(:20437-20451).
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, Hashable, Iterator, List, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import host
from .needs import CacheNeed, CacheView
from .pages import CacheAccountingError, OutOfPages, PagePool, SlotPool

NO_PAGE = host.NO_PAGE
_FIRST_NAMED_ID = 1 << 62       # ids of requests whose key is not a small non-negative integer


class _Tables(Mapping):
    """The block tables of one page group: request -> page per block (NO_PAGE once given back)."""

    def __init__(self, manager: "CacheManager", group: int):
        self._manager, self._group = manager, group

    def __getitem__(self, request: Hashable) -> List[int]:
        manager = self._manager
        if request not in manager.requests:
            raise KeyError(request)
        native = manager._id(request)
        capacity = manager.max_pages_per_request
        pages = host.ints(capacity)
        count = manager._lib.fwh_cache_table(manager._native, native, self._group, pages, capacity)
        if count < 0:
            raise KeyError(request)
        return list(pages[:count])

    def __iter__(self) -> Iterator[Hashable]:
        return iter(self._manager.requests)

    def __len__(self) -> int:
        return len(self._manager.requests)


class _LiveRequests(Mapping):
    """The live requests: key -> (slot, length)."""

    def __init__(self, manager: "CacheManager"):
        self._manager = manager

    def _keys(self) -> List[Hashable]:
        manager = self._manager
        capacity = manager.max_requests
        found = host.ids(capacity)
        count = manager._lib.fwh_cache_live(manager._native, found, capacity)
        return [manager._key(found[i]) for i in range(count)]

    def __contains__(self, request) -> bool:
        manager = self._manager
        native = manager._id(request, create=False)
        return native is not None and bool(manager._lib.fwh_cache_is_live(manager._native, native))

    def __getitem__(self, request: Hashable) -> Tuple[int, int]:
        if request not in self:
            raise KeyError(request)
        return self._manager.slot_of(request), self._manager.length_of(request)

    def __iter__(self) -> Iterator[Hashable]:
        return iter(self._keys())

    def __len__(self) -> int:
        manager = self._manager
        return manager._lib.fwh_cache_live(manager._native, host.ids(0), 0)


@dataclass
class PageGroup:
    key: Tuple
    need: CacheNeed
    entries: List[int]
    pool: PagePool
    tables: Mapping


class CacheManager:
    def __init__(self, needs: Mapping[int, object], num_pages, max_requests: int, page_size: int = 64,
                 max_pages_per_request: Optional[int] = None, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None):
        """``needs``: cache entry id -> a :class:`CacheNeed` (``PagedKV``, ``FixedState`` or a
        class of the mixer's own). ``num_pages``: pages of every page group, or a mapping from a
        group's key (``need.group_key()``) to the pages of that group, with ``None`` as the key of
        all others: a group that keeps a window of keys needs far fewer pages than one that keeps
        them all. ``device`` None keeps the bookkeeping only (no storage)."""
        self.page_size = page_size
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = device
        self.groups: List[PageGroup] = []
        self.entry_group: Dict[int, int] = {}
        self.state_entries: Dict[int, CacheNeed] = {}
        self.needs: Dict[int, CacheNeed] = {}
        grouped: Dict[Tuple, Tuple[CacheNeed, List[int]]] = {}
        for entry in sorted(needs):
            need = needs[entry]
            if need is None:
                continue
            if not isinstance(need, CacheNeed):
                raise TypeError(f"cache entry {entry}: {need!r} is not a CacheNeed")
            self.needs[entry] = need
            if need.paged:
                grouped.setdefault(need.group_key(), (need, []))[1].append(entry)
                self.entry_group[entry] = list(grouped).index(need.group_key())
            else:
                self.state_entries[entry] = need
        # pages of each group
        if isinstance(num_pages, Mapping):
            unknown = [key for key in num_pages if key is not None and key not in grouped]
            if unknown:
                raise ValueError(f"pages are given for page groups that do not exist: {unknown}; the groups are {list(grouped)}")
            missing = [key for key in grouped if key not in num_pages and None not in num_pages]
            if missing:
                raise ValueError(f"no number of pages is given for the page groups {missing}")
            self.group_pages = [int(num_pages[key] if key in num_pages else num_pages[None]) for key in grouped]
            default_pages = int(num_pages[None]) if None in num_pages else max(self.group_pages, default=1)
        else:
            self.group_pages = [int(num_pages)] * len(grouped)
            default_pages = int(num_pages)
        # what bounds one sequence: the smallest pool among the groups that keep every key
        keeping_all = [pages for pages, (need, _) in zip(self.group_pages, grouped.values()) if not need.window]
        self.num_pages = min(keeping_all) if keeping_all else (max(self.group_pages) if self.group_pages else default_pages)
        self.max_pages_per_request = max_pages_per_request or max(self.group_pages, default=default_pages)
        # the bookkeeping lives in the host library
        self._lib = host.library()
        windows = (ctypes.c_int * max(len(grouped), 1))(*[int(need.window or 0) for need, _ in grouped.values()])
        if grouped:
            pages = (ctypes.c_int * len(grouped))(*self.group_pages)
            self._native = self._lib.fwh_cache_create_sized(len(grouped), windows, pages, max_requests, page_size,
                                                            self.max_pages_per_request)
        else:
            self._native = self._lib.fwh_cache_create(0, windows, default_pages, max_requests, page_size, self.max_pages_per_request)
        if not self._native:
            raise ValueError(host.last_error())
        for index, (key, (need, entries)) in enumerate(grouped.items()):
            pool = PagePool(borrowed=self._lib.fwh_cache_group_pool(self._native, index), owner=self)
            self.groups.append(PageGroup(key, need, entries, pool, _Tables(self, index)))
        self.slots = SlotPool(borrowed=self._lib.fwh_cache_slot_pool(self._native), owner=self)
        self.requests = _LiveRequests(self)
        self._ids: Dict[Hashable, int] = {}         # keys that are not small integers -> ids of the host library
        self._keys: Dict[int, Hashable] = {}
        self._next_named = _FIRST_NAMED_ID
        # One page of every group and one slot lie behind those the pools hand out: rows that only fill
        # a step up to a size it was recorded for (see Stepper.planned_decode) write there, and nobody
        # reads it.
        self.spare_pages = list(self.group_pages)
        self.spare_slot = max_requests
        # storage: each need allocates its own
        self.storage: Dict[int, object] = {}
        self._state_together: List[Tuple[CacheNeed, object]] = []   # (need, what stands for its entries' storages)
        if device is not None:
            for entry, need in self.needs.items():
                if need.paged:
                    self.storage[entry] = need.allocate(self.group_pages[self.entry_group[entry]] + 1, page_size, dtype, device)
            alike: List[Tuple[CacheNeed, List[int]]] = []       # fixed-size entries whose needs are equal
            for entry, need in self.state_entries.items():
                for other, entries in alike:
                    if type(other) is type(need) and other == need:
                        entries.append(entry)
                        break
                else:
                    alike.append((need, [entry]))
            for need, entries in alike:
                storages, together = need.allocate_together(len(entries), max_requests + 1, page_size, dtype, device)
                self.storage.update(zip(entries, storages))
                self._state_together.append((need, together))

    def view(self, entry: int, block_table=None, writes: bool = True):
        """What the mixer that uses cache entry ``entry`` sees of it."""
        return self.needs[entry].view(self.storage[entry], block_table, writes)

    # the tensors of the built-in needs, by entry
    @property
    def k_pages(self) -> Dict[int, torch.Tensor]:
        return {entry: self.view(entry).k_pages for entry in self.entry_group if entry in self.storage}

    @property
    def v_pages(self) -> Dict[int, torch.Tensor]:
        return {entry: self.view(entry).v_pages for entry in self.entry_group if entry in self.storage}

    @property
    def state(self) -> Dict[int, torch.Tensor]:
        return {entry: self.view(entry).state for entry in self.state_entries if entry in self.storage}

    def __del__(self):
        if getattr(self, "_native", None):
            self._lib.fwh_cache_destroy(self._native)
            self._native = None

    # ----- request keys ---------------------------------------------------------------------
    def _id(self, request: Hashable, create: bool = True) -> Optional[int]:
        """The host library names requests by 64-bit integers: a small non-negative integer key
        is its own id (the scheduler's ids are such), any other key gets one of its own."""
        if isinstance(request, (int, np.integer)) and not isinstance(request, bool) and 0 <= int(request) < _FIRST_NAMED_ID:
            return int(request)
        found = self._ids.get(request)
        if found is None and create:
            found = self._ids[request] = self._next_named
            self._keys[found] = request
            self._next_named += 1
        return found

    def _key(self, native: int) -> Hashable:
        return self._keys.get(native, native)

    def _forget(self, request: Hashable) -> None:
        native = self._ids.pop(request, None)
        if native is not None:
            self._keys.pop(native, None)

    @property
    def native_handle(self):
        """The host library's cache object (for the scheduler, which lives beside it)."""
        return self._native

    # ----- sizes ------------------------------------------------------------------------
    def pages_for(self, tokens: int) -> int:
        return (tokens + self.page_size - 1) // self.page_size

    def pages_missing(self, request: Hashable, new_length: int) -> Dict[int, int]:
        """Per group: pages a reservation up to ``new_length`` would have to take."""
        native = self._id(request, create=False)
        out = host.ints(len(self.groups))
        self._lib.fwh_cache_pages_missing(self._native, -1 if native is None else native, int(new_length), out)
        return {index: out[index] for index in range(len(self.groups))}

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
        slot = self._lib.fwh_cache_admit(self._native, self._id(request))
        if slot == host.OUT_OF_PAGES:
            raise OutOfPages("out of request slots")
        if slot < 0:
            raise CacheAccountingError(host.last_error())
        self.start_slot(slot)
        return slot

    def start_slot(self, slot: int) -> None:
        """A slot's state is what a request starts with (zero, unless the need says otherwise)
        for the request that takes it."""
        for need, together in self._state_together:
            need.initial_together(together, slot)

    def slot_of(self, request: Hashable) -> int:
        slot = self._lib.fwh_cache_slot_of(self._native, self._live_id(request))
        if slot < 0:
            raise KeyError(request)
        return slot

    def length_of(self, request: Hashable) -> int:
        length = self._lib.fwh_cache_length_of(self._native, self._live_id(request))
        if length < 0:
            raise KeyError(request)
        return length

    def _live_id(self, request: Hashable) -> int:
        native = self._id(request, create=False)
        if native is None:
            raise KeyError(f"request {request!r} is not live")
        return native

    def reserve(self, request: Hashable, new_length: int) -> None:
        """Map pages for positions < new_length in every group, or raise OutOfPages and
        change nothing."""
        if request not in self.requests:
            raise KeyError(f"request {request!r} is not live")
        status = self._lib.fwh_cache_reserve(self._native, self._id(request), int(new_length))
        if status == host.OUT_OF_PAGES:
            raise OutOfPages(host.last_error().replace(f"request {self._id(request)} ", f"request {request!r} "))
        if status < 0:
            raise CacheAccountingError(host.last_error())

    # ----- a whole step at once (one call into the host library each) ------------------------------
    # ``natives``: what ``natives_of`` gave for the same requests, so that a step that makes
    # several of these calls translates its request keys once.
    def natives_of(self, requests: Sequence[Hashable]):
        """The host library's ids of these requests (-1 for one it has never seen), as a C array."""
        small = _FIRST_NAMED_ID
        if all(type(r) is int and 0 <= r < small for r in requests):
            return (ctypes.c_int64 * max(len(requests), 1))(*requests)
        natives = host.ids(len(requests))
        for i, request in enumerate(requests):
            native = self._id(request, create=False)
            natives[i] = -1 if native is None else native
        return natives

    def describe(self, requests: Sequence[Hashable], natives=None) -> Tuple[List[int], List[int]]:
        """(lengths, slots) of live requests; KeyError names the first one that is not live."""
        count = len(requests)
        lengths, slots = host.ints(count), host.ints(count)
        natives = self.natives_of(requests) if natives is None else natives
        if self._lib.fwh_cache_describe(self._native, natives, count, lengths, slots) < 0:
            raise KeyError(next((r for r in requests if r not in self.requests), host.last_error()))
        return lengths[:count], slots[:count]

    def reserve_all(self, requests: Sequence[Hashable], new_lengths: Sequence[int], natives=None, count=None) -> None:
        """The reservations of a whole step: all of them, or OutOfPages and nothing changed.
        (``natives`` with ``count``: the requests by the host library's ids alone.)"""
        count = len(requests) if count is None else count
        natives = self.natives_of(requests) if natives is None else natives
        status = self._lib.fwh_cache_reserve_batch(self._native, natives, (ctypes.c_int * max(count, 1))(*new_lengths), count)
        if status == host.OUT_OF_PAGES:
            raise OutOfPages(host.last_error())
        if status < 0:
            raise KeyError(host.last_error())

    def commit_all(self, requests: Sequence[Hashable], new_lengths: Sequence[int], natives=None) -> None:
        count = len(requests)
        natives = self.natives_of(requests) if natives is None else natives
        if self._lib.fwh_cache_commit_batch(self._native, natives, (ctypes.c_int * max(count, 1))(*new_lengths), count) < 0:
            raise ValueError(host.last_error())

    def commit(self, request: Hashable, new_length: int) -> None:
        if request not in self.requests:
            raise KeyError(request)
        if self._lib.fwh_cache_commit(self._native, self._id(request), int(new_length)) < 0:
            raise ValueError(host.last_error())

    def truncate(self, request: Hashable, token_count: int) -> None:
        """Gives back the pages behind the first ``token_count`` tokens in every group (the
        reference's truncate_tokens, native/src/paged_kv.h:180-187): reservations a step did not
        use after all, or a sequence cut back. Fixed-size state cannot be rewound, so a model that
        keeps any can only drop reservations, never tokens it has run."""
        if request not in self.requests:
            raise KeyError(f"request {request!r} is not live")
        if self.state_entries and token_count < self.length_of(request):
            raise CacheAccountingError(f"request {request!r} holds fixed-size state of {self.length_of(request)} tokens, "
                                       f"which cannot be cut back to {token_count}")
        if self._lib.fwh_cache_truncate(self._native, self._id(request), int(token_count)) < 0:
            raise CacheAccountingError(host.last_error())

    def drop_reservations(self, requests: Sequence[Hashable], natives=None) -> None:
        """After a step that did not run: the pages reserved for it beyond each request's
        length go back to the pools."""
        count = len(requests)
        natives = self.natives_of(requests) if natives is None else natives
        lengths, _ = self.describe(requests, natives)
        if self._lib.fwh_cache_truncate_batch(self._native, natives, (ctypes.c_int * max(count, 1))(*lengths), count) < 0:
            raise CacheAccountingError(host.last_error())

    def release(self, request: Hashable) -> None:
        if request not in self.requests:
            raise CacheAccountingError(f"request {request!r} is released but not live")
        if self._lib.fwh_cache_release(self._native, self._id(request)) < 0:
            raise CacheAccountingError(host.last_error())
        self._forget(request)

    # ----- views for the step function ---------------------------------------------------
    def block_table_rows(self, group_index: int, requests: Sequence[Hashable], stride: Optional[int] = None,
                         natives=None, count=None) -> np.ndarray:
        if natives is None:
            natives = self.natives_of(requests)
        count = len(requests) if count is None else count
        if stride is None:
            stride = max(self._lib.fwh_cache_longest_table(self._native, group_index, natives, count), 1)
        rows = np.zeros((count, stride), dtype=np.int32)
        if self._lib.fwh_cache_fill_tables(self._native, group_index, natives, count, stride, rows.ctypes.data) < 0:
            for request in requests:
                if request not in self.requests:
                    raise KeyError(f"request {request!r} is not live")
            raise CacheAccountingError(host.last_error())
        return rows

    # ----- accounting -------------------------------------------------------------------
    def check_invariants(self) -> None:
        """No page lost, none held twice; slots likewise."""
        if self._lib.fwh_cache_check(self._native) < 0:
            raise CacheAccountingError(host.last_error())

    def stats(self) -> Dict[str, int]:
        return {
            "pages_total": self.num_pages,        # of the tightest group that keeps every key
            "pages_free": self.free_pages() if self.groups else self.num_pages,
            "pages_peak": max((g.pool.peak_in_use for g in self.groups), default=0),
            "slots_free": self.slots.free_count,
            "live_requests": len(self.requests),
        }
