"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; groups with and without a window; slots of fixed-size state."""
import random

import numpy as np
import pytest
import torch

from levanter_amd.cache import NO_PAGE, CacheManager, OutOfPages, OutOfSlots, PagedKv, PagePool, SlotState


def make(n_pages=8, page_size=16, max_seqs=4, max_pages_per_seq=8, window=None, extra=()):
    reqs = [(0, PagedKv(2, 16)), (1, PagedKv(2, 16))]
    if window:
        reqs.append((2, PagedKv(2, 16, window=window)))
    reqs += list(extra)
    return CacheManager(reqs, n_pages=n_pages, page_size=page_size, max_seqs=max_seqs, max_pages_per_seq=max_pages_per_seq)


def test_pool_refuses_double_free_and_counts():
    p = PagePool(3)
    a, b = p.alloc(), p.alloc()
    assert (a, b) == (0, 1) and p.n_free == 1
    p.free(a)
    with pytest.raises(RuntimeError, match="freed twice"):
        p.free(a)
    assert p.alloc() == a  # the page freed last is handed out first
    p.alloc()
    with pytest.raises(OutOfPages):
        p.alloc()
    p.check()


def test_units_with_equal_needs_share_a_group():
    c = make(window=40)
    assert len(c.groups) == 2
    assert c.groups[0].units == [0, 1] and c.groups[1].units == [2] and c.groups[1].requirement.window == 40
    assert c.group_of_unit[1] is c.groups[0]


def test_pages_come_lazily_and_go_back_on_close():
    # as the reference's page table (page_table.py:142-275): a page is taken when a token first lands on it
    c = make()
    h = c.open("a")
    assert h.slot == 0 and c.pages_needed(h, 16) == 1 and c.pages_needed(h, 17) == 2
    c.extend(h, 5)
    c.advance(h, 5)
    assert c.groups[0].pages_held(h.slot) == [0] and h.length == 5
    c.extend(h, 11)
    c.advance(h, 11)  # 16 tokens: still one page
    assert c.groups[0].pages_held(h.slot) == [0]
    c.extend(h, 1)
    c.advance(h, 1)
    assert c.groups[0].pages_held(h.slot) == [0, 1]
    assert c.destination(c.groups[0], h, 16) == 1 * 16 + 0 and c.destination(c.groups[0], h, 7) == 7
    c.check_invariants()
    c.close(h)
    assert c.groups[0].pool.n_free == 8 and (c.groups[0].block_tables == NO_PAGE).all()
    with pytest.raises(RuntimeError, match="closed twice"):
        c.close(h)
    c.check_invariants()


def test_extend_is_all_or_nothing():
    c = make(n_pages=3, window=1000)
    a, b = c.open("a"), c.open("b")
    c.extend(a, 32)
    c.advance(a, 32)
    before = [g.pool.n_free for g in c.groups]
    assert not c.can_extend(b, 40)
    with pytest.raises(OutOfPages):
        c.extend(b, 40)
    assert [g.pool.n_free for g in c.groups] == before
    assert all(g.pages_held(b.slot) == [] for g in c.groups)
    c.check_invariants()
    with pytest.raises(ValueError, match="max_pages_per_seq"):
        c.extend(a, 16 * 8)


def test_slots_run_out_and_come_back():
    c = make(max_seqs=2)
    a, b = c.open("a"), c.open("b")
    with pytest.raises(OutOfSlots):
        c.open("c")
    c.close(a)
    assert c.open("c").slot == a.slot


def test_window_group_gives_pages_back_while_the_request_runs():
    c = make(n_pages=6, window=20, max_pages_per_seq=32)
    g_all, g_win = c.groups
    h = c.open("a")
    held = []
    for _ in range(80):  # one token at a time up to 80 tokens
        c.extend(h, 1)
        c.advance(h, 1)
        c.check_invariants()
        held.append(len(g_win.pages_held(h.slot)))
    assert len(g_all.pages_held(h.slot)) == 5
    assert max(held) <= 3  # 20 keys span at most 3 pages of 16
    # the next query (position 80) reads keys 61..80: blocks 0..2 are gone, block 3 (48..63) is still there
    assert (g_win.block_tables[h.slot, :3] == NO_PAGE).all() and g_win.block_tables[h.slot, 3] != NO_PAGE
    c.close(h)
    c.check_invariants()
    assert g_win.pool.n_free == 6


def test_state_slots_are_zeroed_on_admission():
    c = make(extra=[(5, SlotState((3, 2)))])
    c.allocate_tensors(torch.float32, "cpu")
    assert c.state.tensors[5].shape == (4, 3, 2)
    a = c.open("a")
    c.state.tensors[5][a.slot] += 7
    c.close(a)
    b = c.open("b")
    assert b.slot == a.slot and float(c.state.tensors[5][b.slot].abs().sum()) == 0.0
    k, v, g = c.unit_pages(1)
    assert k.shape == (8, 2 * 16 * 16) and g is c.groups[0]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_keep_the_books(seed):
    rng = random.Random(seed)
    c = make(n_pages=12, max_seqs=4, max_pages_per_seq=6, window=24 if seed % 2 else None)
    live = {}
    n_out_of_pages = 0
    for step in range(400):
        op = rng.random()
        if op < 0.25 and c.n_free_slots:
            h = c.open(step)
            live[step] = h
        elif op < 0.85 and live:
            h = live[rng.choice(list(live))]
            n = rng.choice([1, 1, 1, 2, 7, 16, 33])
            if h.length + n > 16 * 6:
                continue
            try:
                c.extend(h, n)
                c.advance(h, n)
            except OutOfPages:
                n_out_of_pages += 1
        elif live:
            c.close(live.pop(rng.choice(list(live))))
        c.check_invariants()
        for g in c.groups:
            held = sum(len(g.pages_held(s)) for s in range(c.max_seqs))
            assert held + g.pool.n_free == g.pool.n_pages  # no page lost
            pages = [p for s in range(c.max_seqs) for p in g.pages_held(s)]
            assert len(pages) == len(set(pages))  # none held twice
    assert n_out_of_pages > 0  # the pool was small enough to run out
    c.reset()
    c.check_invariants()
    assert all(g.pool.n_free == g.pool.n_pages for g in c.groups) and c.n_free_slots == 4


# ---- how many pages each group gets -------------------------------------------------------------------------------
def test_pages_per_group_fixed_none_and_windowed():
    from levanter_amd.cache import pages_per_group

    full, win = (PagedKv(2, 32), 3), (PagedKv(2, 32, window=40), 2)
    kw = dict(page_size=16, max_seqs=4, max_pages_per_seq=64, longest_portion=100, itemsize=2)
    assert pages_per_group([full], max_pages=None, **kw) == [4 * 64]
    assert pages_per_group([full], max_pages=50, **kw) == [50]
    # a window of 40 keys and portions of up to 100 tokens touch ceil(140 / 16) + 1 = 10 pages a request
    assert pages_per_group([full, win], max_pages=None, **kw) == [256, 40]
    assert pages_per_group([full, win], max_pages=30, **kw) == [30, 30]  # never more than was asked for
    assert pages_per_group([(PagedKv(2, 32, window=5000), 1)], max_pages=None, **kw) == [256]  # nor than the tables hold


def test_pages_per_group_auto_takes_what_the_weights_left():
    from levanter_amd.cache import pages_per_group
    from levanter_amd.cache.sizing import GIB, group_page_bytes

    full, win = (PagedKv(8, 128), 32), (PagedKv(8, 128, window=1024), 4)
    kw = dict(page_size=16, max_seqs=64, max_pages_per_seq=512, longest_portion=2048, itemsize=2)
    pb_full, pb_win = group_page_bytes(*full, 16, 2), group_page_bytes(*win, 16, 2)
    assert pb_full == 2 * 32 * 8 * 128 * 16 * 2
    free = 40 * GIB
    got = pages_per_group([full, win], max_pages="auto", free_bytes=lambda: free, reserve_bytes=8 * GIB, **kw)
    n_win = 64 * ((1024 + 2048 + 15) // 16 + 1)
    assert got[1] == n_win
    assert got[0] == (free - 8 * GIB - n_win * pb_win) // pb_full
    assert got[0] * pb_full + got[1] * pb_win <= free - 8 * GIB < (got[0] + 1) * pb_full + got[1] * pb_win
    # plenty of memory: no more than every request at full length
    assert pages_per_group([full], max_pages="auto", free_bytes=lambda: 10_000 * GIB, **kw) == [64 * 512]
    # too little for one request of full length beside the reserve: an error that says how much is needed
    with pytest.raises(MemoryError, match="GiB are free"):
        pages_per_group([full], max_pages="auto", free_bytes=lambda: 8 * GIB + GIB // 2, reserve_bytes=8 * GIB, **kw)
    with pytest.raises(ValueError, match="query"):
        pages_per_group([full], max_pages="auto", **kw)


def test_engine_cache_sized_from_a_stubbed_memory_query():
    from levanter_amd.config import InferenceEngineConfig, LmConfig
    from levanter_amd.engine.loading import make_cache
    from levanter_amd.cache.sizing import GIB
    from tiny_configs import TINY_B

    class Model:  # what make_cache asks of a model
        def cache_requirements(self):
            spec = LmConfig.from_dict(TINY_B).model_spec()
            return [(e.cache, PagedKv(3, 32)) for e in spec.plan]

    cfg = InferenceEngineConfig(max_pages="auto", max_seqs=64, max_pages_per_seq=4096, page_size=16, compute_dtype="float32",
                                cache_memory_reserve_gib=1.0)
    cache = make_cache(Model(), cfg, free_bytes=lambda: 3 * GIB)
    page_bytes = 2 * 3 * 3 * 32 * 16 * 4  # keys and values, 3 layers, 3 heads of 32, 16 tokens, float32
    assert [g.pool.n_pages for g in cache.groups] == [2 * GIB // page_bytes]
    with pytest.raises(Exception, match="auto"):
        InferenceEngineConfig(max_pages="most")


def test_padding_tokens_of_a_replayed_step_beside_a_window_that_has_moved_on():
    """Steps of single tokens are filled up to a multiple of 8 with padding tokens (request row 0, position 0, written
    nowhere). In a group with a window the first request's block 0 has long been given back: the padding names a
    block without a page, which the attention kernels mask. Every key that a real token can see has a page."""
    import torch

    from levanter_amd.engine.step import ModelRunner, StepEntry, graph_batch_bucket
    from levanter_amd.parts import BuildEnv
    from levanter_amd.parts.spec import PlanEntry

    class Model:
        vocab_size, max_positions, plan = 50, None, [PlanEntry(0, 0), PlanEntry(1, 1)]

        def cache_requirements(self):
            return [(0, PagedKv(1, 16)), (1, PagedKv(1, 16, window=20))]

    window = 20
    cache = CacheManager(Model().cache_requirements(), n_pages=[40, 16], page_size=16, max_seqs=8, max_pages_per_seq=8)
    runner = ModelRunner(Model(), cache, BuildEnv(torch.float32, torch.device("cpu"), None), allocate=False)
    handles = [cache.open(i) for i in range(5)]
    for h in handles:
        cache.extend(h, 60)
        cache.advance(h, 60)
    assert cache.groups[1].block_tables[handles[0].slot, 0] == NO_PAGE  # behind the window
    entries = [StepEntry(h, [7], [0]) for h in handles]
    for h in handles:
        cache.extend(h, 1)
    b = runner._build_host(entries, pad_blocks=1, pad_batch=True)
    assert b.n_tokens == graph_batch_bucket(5) == 8 and b.n_rows_real == 5
    view = lambda i: b.host[b.offs[i]:b.offs[i] + b.sizes[i]]
    positions, token_seq = view(1), view(2)
    assert list(positions[5:]) == [0, 0, 0] and list(token_seq[5:]) == [0, 0, 0]
    for gi, g in enumerate(cache.groups):
        bt = view(8 + 2 * gi).reshape(b.n_seqs, b.max_blocks)
        dest = view(9 + 2 * gi)
        assert (dest[:5] >= 0).all() and (dest[5:] == -1).all()
        w = g.requirement.window
        for t in range(5):  # real tokens: every visible key has a page
            lo = 0 if w is None else max(0, positions[t] - w + 1)
            assert (bt[token_seq[t], lo // 16: positions[t] // 16 + 1] != NO_PAGE).all()
    assert list(view(7)) == [h.slot for h in handles] + [-1, -1, -1]  # padding tokens belong to no slot
    assert view(8 + 2 * 1).reshape(b.n_seqs, b.max_blocks)[0, 0] == NO_PAGE  # what the padding tokens point at
