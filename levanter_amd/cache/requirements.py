"""What a mixer asks of the cache manager. A mixer returns one of these from
``cache_requirement()`` (or None); cache units with equal requirements form a group."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class PagedKv:
    """Keys and values of every past token (or of the last ``window`` tokens), in pages."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None  # None: all keys. w: a query at position p reads keys p-w+1 .. p


@dataclass(frozen=True)
class SlotState:
    """A tensor of fixed shape per live request, zeroed when the request is admitted."""

    shape: Tuple[int, ...]
    dtype: str = "float32"
