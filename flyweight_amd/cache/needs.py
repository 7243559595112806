"""What per-request memory a mixer asks of the cache manager.

A need is an object of a class derived from :class:`CacheNeed`. It says whether the memory
grows with the sequence (``paged``: the entry joins a page group, gets pages through a block
table) or is of fixed size per request (a slot), how it is stored (``allocate``), what a
request starts with (``initial``) and what a mixer sees of it during a step (``view``). The
cache manager asks these questions and nothing else, so a mixer may bring a need class of its
own: a compressed or latent cache, a state that does not start at zero.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Tuple

import torch

from ..kernels import ops


@dataclass
class CacheView:
    """What a mixer sees of the cache during one execution. A need class of another kind may
    return any object of its own from ``view`` instead."""
    k_pages: Optional[torch.Tensor] = None
    v_pages: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None     # [segments, stride] int32, rows in batch order
    state: Optional[torch.Tensor] = None           # [slots, ...]
    writes: bool = True


class CacheNeed:
    """Interface of a need. ``paged`` True: ``allocate(units, ...)`` is called with the number of
    pages (the pool's pages and one spare behind them) and ``group_key()`` / ``window`` sort the
    entry into a page group; entries with equal keys share one pool and one block table per
    request. ``paged`` False: ``allocate`` is called with the number of slots (the most live
    requests and one spare), and ``initial(storage, slot)`` is called whenever a slot is handed
    to a new request."""

    paged: bool = False
    window: Optional[int] = None

    def group_key(self) -> Tuple:
        raise NotImplementedError

    def allocate(self, units: int, page_size: int, dtype: torch.dtype, device: torch.device) -> Any:
        """The storage of one cache entry: any object; it is handed back to ``initial`` and ``view``."""
        raise NotImplementedError

    def initial(self, storage: Any, slot: int) -> None:
        """Fixed-size needs: put slot ``slot`` into the state a request starts with."""

    def allocate_together(self, count: int, units: int, page_size: int, dtype: torch.dtype, device: torch.device):
        """Fixed-size needs: the storages of ``count`` cache entries whose needs equal this one, and
        an object that stands for all of them (``initial_together`` gets it). A need that can
        start a slot of all its entries with one launch overrides both; as they stand they go
        entry by entry."""
        storages = [self.allocate(units, page_size, dtype, device) for _ in range(count)]
        return storages, storages

    def initial_together(self, together: Any, slot: int) -> None:
        for storage in together:
            self.initial(storage, slot)

    def view(self, storage: Any, block_table: Optional[torch.Tensor], writes: bool) -> Any:
        raise NotImplementedError


@dataclass(frozen=True)
class PagedKV(CacheNeed):
    """Keys and values that grow with the sequence. Layers whose needs are equal share
    a group: one page pool and one block table per request. ``window`` None keeps all
    keys; a number keeps only the last ``window`` of them, and pages the window has
    passed are given back. K keeps a key's channels together ([page][kv_head][token][channel]:
    the order the scores reduce over), V a channel's tokens ([page][kv_head][channel][token]:
    the order the weighted sum reduces over)."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    paged = True

    def group_key(self) -> Tuple:
        return ("kv", self.num_kv_heads, self.head_dim, self.window)

    def allocate(self, units, page_size, dtype, device):
        return (torch.zeros((units, self.num_kv_heads, page_size, self.head_dim), dtype=dtype, device=device),
                torch.zeros((units, self.num_kv_heads, self.head_dim, page_size), dtype=dtype, device=device))

    def view(self, storage, block_table, writes):
        return CacheView(k_pages=storage[0], v_pages=storage[1], block_table=block_table, writes=writes)


@dataclass(frozen=True)
class FixedState(CacheNeed):
    """State of fixed size per request (a convolution's last inputs, a recurrence's
    matrix): ``shape`` elements of ``dtype``, zero when a request starts."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    paged = False

    def allocate(self, units, page_size, dtype, device):
        return torch.zeros((units, *self.shape), dtype=self.dtype, device=device)

    def initial(self, storage, slot):
        if storage.is_cuda:
            ops.fill_zero(storage[slot])
        else:
            storage[slot].zero_()

    def allocate_together(self, count, units, page_size, dtype, device):
        # one tensor for the layers that keep the same state: a request's start clears its slot in
        # all of them with one launch (a model of 22 such layers paid 22 before every admission)
        whole = torch.zeros((count, units, *self.shape), dtype=self.dtype, device=device)
        return [whole[index] for index in range(count)], whole

    def initial_together(self, together, slot):
        if together.is_cuda:
            ops.fill_zero_pieces(together[0, slot], together.shape[0], together.stride(0) * together.element_size())
        else:
            together[:, slot].zero_()

    def view(self, storage, block_table, writes):
        return CacheView(state=storage, writes=writes)
