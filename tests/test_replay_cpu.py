"""The step function, the cache manager and the batch tables under every way of cutting the work,
on the CPU with the emulated kernels: what differs from the plain implementation here is a fault
of the host logic, not of a kernel."""
import pytest
import torch

import plain_gpt2 as P
import traces as TR
from emulated_kernels import EmulatedKernels
from helpers import read_weights, write_model
from levanter_amd.config import InferenceEngineConfig
from levanter_amd.engine import ModelRunner, StepEntry, StepError
from levanter_amd.engine.loading import load_model, make_cache
from levanter_amd.parts import BuildEnv
from tiny_configs import TINY


@pytest.fixture(scope="module", params=["A", "B"])
def setup(request):
    raw, seed = TINY[request.param]
    d = write_model(raw, seed, torch.float32)
    env = BuildEnv(torch.float32, torch.device("cpu"), EmulatedKernels())
    _, model = load_model(d, env)
    weights = read_weights(d)
    lengths = [70, 45, 100, 37, 64, 33] if request.param == "A" else [90, 130, 41, 200, 64, 17]
    reqs = TR.random_requests(raw["vocab_size"], lengths, seed + 10)
    plain = {rid: P.plain_logits(weights, raw, torch.tensor(t)) for rid, t in reqs.items()}
    return raw, model, env, reqs, plain


def replay(model, env, steps, max_tokens, slots=None):
    """``slots``: request id -> the slot it must occupy."""
    ps = 16
    cfg = InferenceEngineConfig(max_pages=max_tokens // ps, max_seqs=4, page_size=ps, max_pages_per_seq=16, compute_dtype="float32")
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    live, out = {}, {}
    if slots:  # a fresh manager hands out slots 0, 1, 2 ... in order
        who = {slot: rid for rid, slot in slots.items()}
        opened = [cache.open(who.get(i, ("placeholder", i))) for i in range(max(who) + 1)]
        for h in opened:
            if h.request_id in slots:
                live[h.request_id] = h
            else:
                cache.close(h)
        assert {rid: live[rid].slot for rid in slots} == slots
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in live:
                live[e["id"]] = cache.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        logits = runner.step(entries)
        cache.check_invariants()
        if logits.shape[0]:
            out[s["step"]] = logits
        for rid in s["end"]:
            cache.close(live.pop(rid))
    cache.check_invariants()
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups)
    return out


@pytest.mark.parametrize("mode", ["whole", "singles", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(setup, mode):
    raw, model, env, reqs, plain = setup
    steps = {"whole": TR.trace_whole, "singles": TR.trace_prefill_then_singles, "portions": TR.trace_portions,
             "mixed": lambda r: TR.trace_mixed(r, seed=3)}[mode](reqs)
    TR.number(steps)
    max_tokens = TR.peak_tokens(steps)
    got = replay(model, env, steps, max_tokens)
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    assert set(got) == set(want)
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=1e-4, atol=1e-5)


def test_mixed_trace_really_mixes_and_reuses_pages(setup):
    raw, model, env, reqs, plain = setup
    steps = TR.number(TR.trace_mixed(reqs, seed=3))
    assert any(len(s["entries"]) >= 3 for s in steps)
    assert any(any(len(e["tokens"]) == 1 for e in s["entries"]) and any(len(e["tokens"]) > 1 for e in s["entries"]) for s in steps)
    total = sum((len(t) + 63) // 64 * 64 for t in reqs.values())
    assert TR.peak_tokens(steps) < total  # the pool is smaller than all requests together: pages are used again


def test_step_refuses_bad_input(setup):
    raw, model, env, reqs, plain = setup
    cfg = InferenceEngineConfig(max_pages=8, max_seqs=2, page_size=16, max_pages_per_seq=32, compute_dtype="float32")
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    h = cache.open("a")
    with pytest.raises(StepError, match="outside the vocabulary"):
        runner.step([StepEntry(h, [raw["vocab_size"]], [0])])
    with pytest.raises(StepError, match="wanted place"):
        runner.step([StepEntry(h, [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry(h, [1], []), StepEntry(h, [2], [])])
    with pytest.raises(StepError, match="no tokens"):
        runner.step([StepEntry(h, [], [])])
    with pytest.raises(StepError, match="limit"):  # beyond the position table
        runner.step([StepEntry(h, [1] * (raw["n_positions"] + 1), [])])
    assert h.length == 0 and all(g.pool.n_free == 8 for g in cache.groups)  # nothing changed
    from levanter_amd.cache import OutOfPages

    h2 = cache.open("b")
    runner.step([StepEntry(h, [1] * 100, [])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry(h2, [1] * 40, [0])])
    assert h2.length == 0
    cache.check_invariants()
    assert runner.step([]).shape == (0, raw["vocab_size"])


def test_token_ids_from_the_device_for_the_first_entries_of_a_mixed_step(setup):
    """A step may take the token ids of its first entries (single tokens) from a tensor on the device, in any order
    of its rows, beside a prompt portion given on the host: the logits equal those of the same step with all ids
    given; fed ids for an entry of several tokens, or for more entries than the step has, are refused."""
    raw, model, env, reqs, plain = setup
    cfg = InferenceEngineConfig(max_pages=32, max_seqs=4, page_size=16, max_pages_per_seq=16, compute_dtype="float32")
    toks = list(reqs.values())

    def run(feed):
        cache = make_cache(model, cfg)
        runner = ModelRunner(model, cache, env)
        a, b, c = cache.open("a"), cache.open("b"), cache.open("c")
        runner.step([StepEntry(a, toks[0][:20], []), StepEntry(b, toks[1][:7], [])])
        ids = [toks[0][20], toks[1][7]]
        entries = [StepEntry(a, [0] if feed else [ids[0]], [0]), StepEntry(b, [0] if feed else [ids[1]], [0]),
                   StepEntry(c, toks[2][:9], [8])]
        if not feed:
            return runner.step(entries)
        sampled = torch.tensor([5, ids[1], 7, ids[0]], dtype=torch.int32)  # rows of another step's sampler output
        with pytest.raises(StepError, match="first entries"):
            runner.step(entries, token_feed=(sampled, torch.tensor([3, 1, 0]), 3))
        with pytest.raises(StepError, match="first entries"):
            runner.step(entries, token_feed=(sampled, torch.tensor([3, 1, 0, 2]), 4))
        assert a.length == 20 and c.length == 0  # a refused step changes nothing
        return runner.step(entries, token_feed=(sampled, torch.tensor([3, 1]), 2))

    torch.testing.assert_close(run(True), run(False), rtol=0, atol=0)


def test_a_step_that_fails_in_the_model_gives_its_pages_back(setup, monkeypatch):
    raw, model, env, reqs, plain = setup
    cfg = InferenceEngineConfig(max_pages=16, max_seqs=2, page_size=16, max_pages_per_seq=16, compute_dtype="float32")
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    toks = list(reqs.values())[0]
    a, b = cache.open("a"), cache.open("b")
    runner.step([StepEntry(a, toks[:20], [])])
    free = [g.pool.n_free for g in cache.groups]
    real_forward = model.forward

    def broken(ctx, rows):
        raise RuntimeError("a part failed")

    monkeypatch.setattr(model, "forward", broken)
    with pytest.raises(RuntimeError, match="a part failed"):
        runner.step([StepEntry(a, toks[20:45], [24]), StepEntry(b, toks[:33], [])])
    assert a.length == 20 and b.length == 0 and [g.pool.n_free for g in cache.groups] == free
    cache.check_invariants()
    monkeypatch.setattr(model, "forward", real_forward)
    got = runner.step([StepEntry(a, toks[20:45], [24]), StepEntry(b, toks[:33], [])])
    torch.testing.assert_close(got[0].double(), plain[list(reqs)[0]][44], rtol=1e-4, atol=1e-5)
    cache.close(a)
    cache.close(b)
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups)


def test_the_reference_s_ragged_schedule(setup):
    """tests/inference/test_paged_attention.py:378-442: two requests of 8 tokens filled by [[4,2],[0,1],[0,1],[2,1],[1,2],[1,1]]
    tokens a step (a request is left out where its count is 0); every step's rows equal the whole sequence's."""
    raw, model, env, reqs, plain = setup
    t0, t1 = reqs["r0"][:8], reqs["r1"][:8]
    steps = TR.trace_two_requests(t0, t1, TR.REFERENCE_RAGGED_SCHEDULE)
    got = replay(model, env, steps, 128)
    want = TR.expected_rows(steps, lambda rid: plain["r0" if rid == "a" else "r1"])
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("slots", TR.REFERENCE_SLOT_ORDERS)
@pytest.mark.parametrize("chunk", TR.REFERENCE_CHUNK_SIZES)
def test_the_reference_s_chunked_prefill_in_every_slot_order(setup, slots, chunk):
    """tests/inference/test_paged_attention.py:293-376: a prefix of 1, 2 or 3 tokens of two requests, then four chunks of
    1, 2, 3 or 8 tokens each, with the requests in slots [0,1], [1,0], [2,0], [0,2], [2,1]."""
    raw, model, env, reqs, plain = setup
    for prefix in TR.REFERENCE_PREFIX_SIZES:
        n = prefix + 4 * chunk
        steps = TR.trace_two_requests(reqs["r0"][:n], reqs["r1"][:n], TR.reference_chunk_schedule(prefix, chunk))
        got = replay(model, env, steps, 128, slots={"a": slots[0], "b": slots[1]})
        want = TR.expected_rows(steps, lambda rid: plain["r0" if rid == "a" else "r1"])
        for k in want:
            torch.testing.assert_close(got[k].double(), want[k], rtol=1e-4, atol=1e-5)
