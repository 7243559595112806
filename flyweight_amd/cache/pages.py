"""Page pool, block tables and state slots: the bookkeeping of the cache, host side.

A page holds ``page_size`` consecutive tokens of one sequence. The pool is a LIFO stack
of free page ids, so a page given back is the next one handed out; a sequence's block
table maps token t to page ``table[t // page_size]``. Same operations as the reference's
(unwired) primitive: native/src/paged_kv.h:133-204 (pool, ensure/truncate/release).
"""

from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """The pool cannot cover a reservation; nothing was allocated."""


class CacheAccountingError(AssertionError):
    """A page or slot was freed twice, or freed without being held."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # pop() hands out page 0 first
        self._held = [False] * num_pages
        self.peak_in_use = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def in_use(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("out of cache pages")
        page = self._free.pop()
        self._held[page] = True
        self.peak_in_use = max(self.peak_in_use, self.in_use)
        return page

    def free(self, page: int) -> None:
        if not 0 <= page < self.num_pages or not self._held[page]:
            raise CacheAccountingError(f"page {page} is freed but not held")
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]


class SlotPool:
    """Slots of fixed-size per-request state; also a LIFO stack."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("a slot pool needs at least one slot")
        self.num_slots = num_slots
        self._free: List[int] = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def free_count(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("out of request slots")
        slot = self._free.pop()
        self._held[slot] = True
        return slot

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._held[slot]:
            raise CacheAccountingError(f"slot {slot} is freed but not held")
        self._held[slot] = False
        self._free.append(slot)
