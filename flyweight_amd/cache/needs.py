"""What per-request memory a mixer asks of the cache manager."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedKV:
    """Keys and values that grow with the sequence. Layers whose needs are equal share
    a group: one page pool and one block table per request. ``window`` None keeps all
    keys; a number keeps only the last ``window`` of them, and pages the window has
    passed are given back."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def group_key(self) -> Tuple:
        return ("kv", self.num_kv_heads, self.head_dim, self.window)


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request (a convolution's last inputs, a recurrence's
    matrix): ``shape`` elements of ``dtype``, zero when a request starts."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
