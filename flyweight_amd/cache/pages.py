"""Page pool and state slots: Python faces of the host library's LIFO pools.

A page holds ``page_size`` consecutive tokens of one sequence. The pool is a LIFO stack
of free page ids, so a page given back is the next one handed out; a sequence's block
table maps token t to page ``table[t // page_size]``. Same operations as the reference's
(unwired) primitive: native/src/paged_kv.h:133-204 (pool, ensure/truncate/release). The
bookkeeping itself is C++ (``csrc/host/cache.hpp``).
"""

from __future__ import annotations

from .. import host


class OutOfPages(RuntimeError):
    """The pool cannot cover a reservation; nothing was allocated."""


class CacheAccountingError(AssertionError):
    """A page or slot was freed twice, or freed without being held."""


class _Pool:
    """A pool of the host library: its own (``size``) or one that lives inside a cache
    (``borrowed`` handle, freed with the cache)."""

    _empty_message = "out of cache pages"
    _what = "page"

    def __init__(self, size: int = 0, borrowed=None, owner=None):
        self._lib = host.library()
        self._owner = owner                 # keeps the cache alive while its pool is looked at
        if borrowed is not None:
            self._handle, self._owned = borrowed, False
        else:
            if size <= 0:
                raise ValueError(f"a {self._what} pool needs at least one {self._what}")
            self._handle, self._owned = self._lib.fwh_pool_create(size), True

    def __del__(self):
        if getattr(self, "_owned", False) and self._handle:
            self._lib.fwh_pool_destroy(self._handle)
            self._handle = None

    @property
    def size(self) -> int:
        return self._lib.fwh_pool_size(self._handle)

    @property
    def free_count(self) -> int:
        return self._lib.fwh_pool_free_count(self._handle)

    @property
    def in_use(self) -> int:
        return self.size - self.free_count

    @property
    def peak_in_use(self) -> int:
        return self._lib.fwh_pool_peak(self._handle)

    def alloc(self) -> int:
        got = self._lib.fwh_pool_alloc(self._handle)
        if got < 0:
            raise OutOfPages(self._empty_message)
        return got

    def free(self, index: int) -> None:
        if self._lib.fwh_pool_free(self._handle, int(index)) < 0:
            raise CacheAccountingError(f"{self._what} {index} is freed but not held")

    def is_held(self, index: int) -> bool:
        return bool(self._lib.fwh_pool_is_held(self._handle, int(index)))


class PagePool(_Pool):
    def __init__(self, num_pages: int = 0, borrowed=None, owner=None):
        super().__init__(num_pages, borrowed, owner)

    @property
    def num_pages(self) -> int:
        return self.size


class SlotPool(_Pool):
    """Slots of fixed-size per-request state; also a LIFO stack."""

    _empty_message = "out of request slots"
    _what = "slot"

    def __init__(self, num_slots: int = 0, borrowed=None, owner=None):
        super().__init__(num_slots, borrowed, owner)

    @property
    def num_slots(self) -> int:
        return self.size
