"""A pool of page ids with reference counts.

The reference keeps ``page_ref_counts`` beside the block tables and takes the free page with
the lowest index (src/levanter/inference/page_table.py:35-39,209-242); pages are never cleared
when they are given back (page_table.py:326-357), reads are bounded by lengths instead. Here
freed pages go on a stack, so the page freed last is handed out first: reuse happens early,
which is what tests of stale data want.
"""
from __future__ import annotations

from typing import List

import numpy as np


class OutOfPages(RuntimeError):
    """The pool has no free page left (the reference's "Out of free pages during allocation",
    page_table.py:219-223)."""


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = int(n_pages)
        self.ref_counts = np.zeros(self.n_pages, dtype=np.int32)
        self._free: List[int] = list(range(self.n_pages - 1, -1, -1))  # pop() gives page 0 first

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("out of free pages")
        page = self._free.pop()
        assert self.ref_counts[page] == 0, f"page {page} was on the free list while held"
        self.ref_counts[page] = 1
        return page

    def share(self, page: int) -> None:
        """One more holder of a page that is already held (kept for cloned requests)."""
        if self.ref_counts[page] <= 0:
            raise RuntimeError(f"page {page} is not held and cannot be shared")
        self.ref_counts[page] += 1

    def free(self, page: int) -> None:
        if not 0 <= page < self.n_pages:
            raise RuntimeError(f"page {page} is outside the pool of {self.n_pages}")
        if self.ref_counts[page] <= 0:
            raise RuntimeError(f"page {page} is freed twice")
        self.ref_counts[page] -= 1
        if self.ref_counts[page] == 0:
            self._free.append(page)

    def check(self) -> None:
        """No page lost, none held and free at once."""
        free = set(self._free)
        assert len(free) == len(self._free), "a page is on the free list twice"
        for p in range(self.n_pages):
            held = self.ref_counts[p] > 0
            assert held != (p in free), f"page {p}: ref count {self.ref_counts[p]} but {'on' if p in free else 'off'} the free list"
