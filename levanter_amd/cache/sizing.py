"""How many pages each cache group's pool gets.

The reference sizes its one pool as ``max_seqs * max_pages_per_seq`` unless ``max_pages`` is given
(src/levanter/inference/engine.py:108-111) and notes sizing from free memory as an open item
(.agents/projects/inference.md:175). Here ``max_pages`` may also be ``"auto"``: the pools take what is left of the
GPU's memory once the weights are there, less a reserve for activations and kernel workspaces.

Groups differ in what they need. A group that keeps every key needs ``max_pages`` pages to hold the same number of
tokens as any other such group. A group with a window needs, per live request, the pages of the window and of the
longest portion a step may bring (pages behind the window go back after each step), however long requests get.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence, Tuple

from .requirements import PagedKv

GIB = 1 << 30


def group_page_bytes(req: PagedKv, n_units: int, page_size: int, itemsize: int) -> int:
    """Bytes of one page of a group: keys and values of ``page_size`` tokens in each of its cache units."""
    return 2 * n_units * req.n_kv_heads * req.head_dim * page_size * itemsize


def window_group_pages(req: PagedKv, page_size: int, max_seqs: int, max_pages_per_seq: int, longest_portion: int) -> int:
    """The most pages a windowed group can hold at once: per live request the blocks that the window and one step's
    portion touch (one more for a window that starts inside a block), never more than a request's table has."""
    per_seq = (req.window + longest_portion + page_size - 1) // page_size + 1
    return max_seqs * min(per_seq, max_pages_per_seq)


def pages_per_group(groups: Sequence[Tuple[PagedKv, int]], *, max_pages, page_size: int, max_seqs: int, max_pages_per_seq: int,
                    longest_portion: int, itemsize: int, free_bytes: Optional[Callable[[], int]] = None,
                    reserve_bytes: int = 8 * GIB) -> List[int]:
    """``groups``: (requirement, number of cache units) per group. ``max_pages``: an int (pages of every group that
    keeps all keys; windowed groups take what they can use of it), None (``max_seqs * max_pages_per_seq``) or "auto"
    (what ``free_bytes()`` less ``reserve_bytes`` holds: windowed groups first, the rest in equal page counts to the
    groups that keep all keys, at most ``max_seqs * max_pages_per_seq``)."""
    most = max_seqs * max_pages_per_seq
    windowed = [None if req.window is None else window_group_pages(req, page_size, max_seqs, max_pages_per_seq, longest_portion)
                for req, _ in groups]
    if max_pages != "auto":
        full = most if max_pages is None else int(max_pages)
        return [full if w is None else min(full, w) for w in windowed]
    if free_bytes is None:
        raise ValueError('max_pages="auto" needs a query of the free device memory')
    budget = int(free_bytes()) - int(reserve_bytes)
    per_page = [group_page_bytes(req, n, page_size, itemsize) for req, n in groups]
    budget -= sum(w * b for w, b in zip(windowed, per_page) if w is not None)
    full_bytes = sum(b for w, b in zip(windowed, per_page) if w is None)
    full = most if full_bytes == 0 else min(most, budget // full_bytes)
    least = max_pages_per_seq  # one request of full length must fit, or nothing can be promised
    if budget < 0 or full < least:
        need = sum(w * b for w, b in zip(windowed, per_page) if w is not None) + least * full_bytes + int(reserve_bytes)
        raise MemoryError(f'max_pages="auto": {int(free_bytes()) / GIB:.1f} GiB are free, but a cache for one request of '
                          f"{max_pages_per_seq} pages and a reserve of {reserve_bytes / GIB:.1f} GiB need {need / GIB:.1f} GiB")
    return [int(full) if w is None else int(w) for w in windowed]
