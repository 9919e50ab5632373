"""The cache manager: pages of keys and values with a block table per request and group, and
slots of fixed-size per-request state.

Reference: ``PageTable`` (src/levanter/inference/page_table.py:26-505) holds ``page_indices
[seq, page]``, ``page_ref_counts``, ``seq_lens`` and ``used_mask``; pages are allocated lazily,
exactly when a token first lands on them (page_table.py:142-275) and freed when a sequence
finishes (:326-403). One page id addresses the same page in every layer
(src/levanter/models/llama.py:427-432). ``DecodeState`` rows are the reference's per-slot state
of fixed size (src/levanter/inference/jit_scheduler.py:66-117).

Differences: the tables live on the host; cache units (one per plan entry that writes a
cache) whose mixers ask for the same thing form a *group* with a pool and block tables of its
own, so that a group that keeps only a window of keys can give pages back while the request
runs; fixed-size state lives in ``StateSlots`` indexed by the request's slot.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .page_pool import OutOfPages, PagePool
from .requirements import PagedKv, SlotState

NO_PAGE = -1

_TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class OutOfSlots(RuntimeError):
    pass


def k_page_elems(req: PagedKv, page_size: int) -> int:
    return req.n_kv_heads * req.head_dim * page_size


class PagedGroup:
    """Cache units with one requirement: a pool, a block table per slot, and the page tensors.

    Device layout of one unit: keys ``[page, kv_head, head_dim/8, page_size, 8]`` (a run of 8
    consecutive head dimensions of one token is contiguous, tokens of a page next to each
    other), values ``[page, kv_head, head_dim, page_size]`` (transposed: the tokens of a page
    are contiguous for one head dimension). Both are what the matrix instructions of the
    attention kernels read without a transposition."""

    def __init__(self, index: int, req: PagedKv, units: List[int], n_pages: int, page_size: int, max_seqs: int,
                 max_pages_per_seq: int):
        self.index = index
        self.requirement = req
        self.units = list(units)
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        self.max_pages_per_seq = max_pages_per_seq
        self.block_tables = np.full((max_seqs, max_pages_per_seq), NO_PAGE, dtype=np.int32)
        self.first_live_block = np.zeros(max_seqs, dtype=np.int32)  # blocks before it were given back (window)
        self.k_pages: Optional[torch.Tensor] = None  # [unit, page, elems]
        self.v_pages: Optional[torch.Tensor] = None
        self.unit_pos = {u: i for i, u in enumerate(self.units)}

    def allocate_tensors(self, dtype: torch.dtype, device) -> None:
        elems = k_page_elems(self.requirement, self.page_size)
        shape = (len(self.units), self.pool.n_pages, elems)
        self.k_pages = torch.zeros(shape, dtype=dtype, device=device)
        self.v_pages = torch.zeros(shape, dtype=dtype, device=device)

    def bytes_per_token(self, itemsize: int) -> int:
        return 2 * len(self.units) * self.requirement.n_kv_heads * self.requirement.head_dim * itemsize

    # ---- per-request bookkeeping -------------------------------------------------
    def blocks_needed(self, slot: int, old_len: int, new_len: int) -> int:
        have = (old_len + self.page_size - 1) // self.page_size
        want = (new_len + self.page_size - 1) // self.page_size
        return max(0, want - have)

    def extend(self, slot: int, old_len: int, new_len: int) -> List[int]:
        """Give pages to blocks ceil(old/ps) .. ceil(new/ps)-1. Returns the new pages (for undo)."""
        have = (old_len + self.page_size - 1) // self.page_size
        want = (new_len + self.page_size - 1) // self.page_size
        if want > self.max_pages_per_seq:
            raise ValueError(f"a request of {new_len} tokens needs {want} pages, more than max_pages_per_seq={self.max_pages_per_seq}")
        got: List[int] = []
        try:
            for b in range(have, want):
                page = self.pool.alloc()
                got.append(page)
                assert self.block_tables[slot, b] == NO_PAGE
                self.block_tables[slot, b] = page
        except OutOfPages:
            for i, page in enumerate(got):
                self.block_tables[slot, have + i] = NO_PAGE
                self.pool.free(page)
            raise
        return got

    def release_behind_window(self, slot: int, length: int) -> int:
        """Give back the pages whose every token is out of reach of any later query.
        The next query stands at position >= length and reads keys > position - window."""
        w = self.requirement.window
        if w is None:
            return 0
        first_needed = max(0, length - w + 1)
        first_block = first_needed // self.page_size
        n = 0
        for b in range(int(self.first_live_block[slot]), first_block):
            page = int(self.block_tables[slot, b])
            if page != NO_PAGE:
                self.pool.free(page)
                self.block_tables[slot, b] = NO_PAGE
                n += 1
        self.first_live_block[slot] = max(int(self.first_live_block[slot]), first_block)
        return n

    def release_all(self, slot: int) -> None:
        row = self.block_tables[slot]
        for b in np.nonzero(row != NO_PAGE)[0]:
            self.pool.free(int(row[b]))
        row[:] = NO_PAGE
        self.first_live_block[slot] = 0

    def pages_held(self, slot: int) -> List[int]:
        row = self.block_tables[slot]
        return [int(p) for p in row[row != NO_PAGE]]


class StateSlots:
    """Fixed-size state per live request for the cache units that ask for it: a tensor
    ``[slot, *shape]`` per unit, zeroed when a request takes the slot."""

    def __init__(self, requirements: Dict[int, SlotState], n_slots: int):
        self.requirements = dict(requirements)
        self.n_slots = n_slots
        self.tensors: Dict[int, torch.Tensor] = {}

    def allocate_tensors(self, device) -> None:
        for unit, req in self.requirements.items():
            self.tensors[unit] = torch.zeros((self.n_slots,) + tuple(req.shape), dtype=_TORCH_DTYPES[req.dtype], device=device)

    def reset_slot(self, slot: int) -> None:
        for t in self.tensors.values():
            t[slot].zero_()


@dataclass
class SequenceHandle:
    """A live request as the cache manager sees it."""

    request_id: object
    slot: int
    length: int = 0  # tokens whose keys and values are in the cache
    closed: bool = False


def group_units(requirements: Sequence[Tuple[int, object]]) -> Tuple[Dict[PagedKv, List[int]], Dict[int, SlotState]]:
    """Sort (cache unit id, requirement) pairs: paged units by requirement (each distinct one is a group, in order of
    first appearance), slot-state units by id."""
    by_req: Dict[PagedKv, List[int]] = {}
    slot_reqs: Dict[int, SlotState] = {}
    for unit, req in requirements:
        if isinstance(req, PagedKv):
            by_req.setdefault(req, []).append(unit)
        elif isinstance(req, SlotState):
            slot_reqs[unit] = req
        elif req is not None:
            raise TypeError(f"cache unit {unit}: unknown cache requirement {req!r}")
    return by_req, slot_reqs


class CacheManager:
    def __init__(self, requirements: Sequence[Tuple[int, object]], *, n_pages, page_size: int, max_seqs: int,
                 max_pages_per_seq: int):
        """``requirements``: (cache unit id, PagedKv | SlotState | None) of every unit. ``n_pages``: pages of every
        group's pool, or one number per group (in the order of ``group_units``)."""
        self.page_size = page_size
        self.max_seqs = max_seqs
        self.max_pages_per_seq = max_pages_per_seq
        by_req, slot_reqs = group_units(requirements)
        counts = [int(n_pages)] * len(by_req) if isinstance(n_pages, (int, np.integer)) else [int(n) for n in n_pages]
        if len(counts) != len(by_req):
            raise ValueError(f"{len(counts)} page counts for {len(by_req)} cache groups")
        self.groups: List[PagedGroup] = [
            PagedGroup(i, req, units, counts[i], page_size, max_seqs, max_pages_per_seq) for i, (req, units) in enumerate(by_req.items())
        ]
        self.group_of_unit: Dict[int, PagedGroup] = {u: g for g in self.groups for u in g.units}
        self.state = StateSlots(slot_reqs, max_seqs)
        self._free_slots: List[int] = list(range(max_seqs - 1, -1, -1))
        self.live: Dict[int, SequenceHandle] = {}  # slot -> handle

    # ---- device memory -------------------------------------------------------------
    def allocate_tensors(self, dtype: torch.dtype, device) -> None:
        for g in self.groups:
            g.allocate_tensors(dtype, device)
        self.state.allocate_tensors(device)

    def unit_pages(self, unit: int) -> Tuple[torch.Tensor, torch.Tensor, PagedGroup]:
        g = self.group_of_unit[unit]
        i = g.unit_pos[unit]
        return g.k_pages[i], g.v_pages[i], g

    # ---- requests --------------------------------------------------------------------
    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    def open(self, request_id) -> SequenceHandle:
        if not self._free_slots:
            raise OutOfSlots("no free request slot")
        slot = self._free_slots.pop()
        h = SequenceHandle(request_id, slot)
        self.live[slot] = h
        if self.state.tensors:
            self.state.reset_slot(slot)
        return h

    def pages_needed(self, h: SequenceHandle, n_new: int) -> int:
        """The most pages any group must still find for ``n_new`` more tokens."""
        return max((g.blocks_needed(h.slot, h.length, h.length + n_new) for g in self.groups), default=0)

    def can_extend(self, h: SequenceHandle, n_new: int) -> bool:
        return all(g.blocks_needed(h.slot, h.length, h.length + n_new) <= g.pool.n_free for g in self.groups)

    def extend(self, h: SequenceHandle, n_new: int) -> None:
        """Make room for tokens ``length .. length+n_new-1`` in every group, or change nothing and raise."""
        assert not h.closed
        if h.length + n_new > self.page_size * self.max_pages_per_seq:
            raise ValueError(
                f"request {h.request_id!r} would hold {h.length + n_new} tokens, more than page_size * max_pages_per_seq = "
                f"{self.page_size * self.max_pages_per_seq}")
        done: List[Tuple[PagedGroup, List[int]]] = []
        try:
            for g in self.groups:
                done.append((g, g.extend(h.slot, h.length, h.length + n_new)))
        except OutOfPages:
            for g, pages in done:
                have = (h.length + self.page_size - 1) // self.page_size
                for i, page in enumerate(pages):
                    g.block_tables[h.slot, have + i] = NO_PAGE
                    g.pool.free(page)
            raise

    def retract(self, h: SequenceHandle, n_new: int) -> None:
        """Undo an ``extend`` whose tokens were never written (the step failed before it ran): the pages of blocks
        beyond the request's length go back to their pools."""
        have = (h.length + self.page_size - 1) // self.page_size
        want = (h.length + n_new + self.page_size - 1) // self.page_size
        for g in self.groups:
            for b in range(have, min(want, g.block_tables.shape[1])):
                page = int(g.block_tables[h.slot, b])
                if page != NO_PAGE:
                    g.block_tables[h.slot, b] = NO_PAGE
                    g.pool.free(page)

    def advance(self, h: SequenceHandle, n_new: int) -> None:
        """The step has written ``n_new`` tokens: count them, give back what windows have passed."""
        h.length += n_new
        for g in self.groups:
            g.release_behind_window(h.slot, h.length)

    def close(self, h: SequenceHandle) -> None:
        if h.closed:
            raise RuntimeError(f"request {h.request_id!r} is closed twice")
        h.closed = True
        for g in self.groups:
            g.release_all(h.slot)
        del self.live[h.slot]
        self._free_slots.append(h.slot)

    def reset(self) -> None:
        for h in list(self.live.values()):
            self.close(h)

    def destination(self, g: PagedGroup, h: SequenceHandle, position: int) -> int:
        page = int(g.block_tables[h.slot, position // self.page_size])
        assert page != NO_PAGE, f"position {position} of request {h.request_id!r} has no page"
        return page * self.page_size + position % self.page_size

    # ---- invariants (tests) ------------------------------------------------------------
    def check_invariants(self) -> None:
        for g in self.groups:
            g.pool.check()
            held: Dict[int, int] = {}
            for slot in range(self.max_seqs):
                pages = g.pages_held(slot)
                if slot not in self.live:
                    assert not pages, f"free slot {slot} holds pages {pages}"
                for p in pages:
                    held[p] = held.get(p, 0) + 1
            for p in range(g.pool.n_pages):
                assert g.pool.ref_counts[p] == held.get(p, 0), (
                    f"group {g.index} page {p}: ref count {g.pool.ref_counts[p]}, in {held.get(p, 0)} block tables")
            for slot, h in self.live.items():
                lo = int(g.first_live_block[slot])
                hi = (h.length + self.page_size - 1) // self.page_size
                row = g.block_tables[slot]
                assert (row[lo:hi] != NO_PAGE).all(), f"slot {slot}: a live block has no page"
                assert (row[:lo] == NO_PAGE).all(), f"slot {slot}: a block behind the window still has a page"
        assert len(set(self._free_slots)) == len(self._free_slots)
        assert set(self._free_slots).isdisjoint(self.live.keys())
        assert len(self._free_slots) + len(self.live) == self.max_seqs
