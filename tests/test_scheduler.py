"""The scheduler's decisions and the engine's bookkeeping, on the CPU: a dummy model with constant
one-hot logits (as the reference's tests/inference/test_engine.py:19-46), the emulated kernels for
sampling, and the real cache manager, step function and scheduler."""
import pytest
import torch

from emulated_kernels import EmulatedKernels
from levanter_amd.cache import PagedKv
from levanter_amd.config import InferenceEngineConfig
from levanter_amd.engine import InferenceEngine, Request, SeqDecodingParams, is_stop_signal
from levanter_amd.parts import BuildEnv
from levanter_amd.parts.spec import PlanEntry


class DummyModel:
    """Keeps pages like a two-layer attention model, computes nothing, prefers token `eos` everywhere
    (or the token after the input token, with ``count=True``)."""

    def __init__(self, vocab_size=10, eos=3, count=False, max_positions=None):
        self.vocab_size = vocab_size
        self.eos = eos
        self.count = count
        self.max_positions = max_positions
        self.plan = [PlanEntry(0, 0), PlanEntry(1, 1)]
        self.batches = []
        self.env = None

    def cache_requirements(self):
        return [(0, PagedKv(1, 16)), (1, PagedKv(1, 16))]

    def forward(self, ctx, rows):
        self.batches.append(list(ctx.host["run_lengths"]))
        n = rows.numel()
        logits = torch.zeros(n, self.vocab_size)
        if self.count:
            nxt = (ctx.tokens[rows.long()].long() + 1) % self.vocab_size
            logits[torch.arange(n), nxt] = 1.0
        else:
            logits[:, self.eos] = 1.0
        return logits


def make_engine(model=None, **kw):
    cfg = InferenceEngineConfig(**{**dict(max_pages=64, max_seqs=8, page_size=16, max_pages_per_seq=4, compute_dtype="float32",
                                          max_seqs_in_prefill=4), **kw})
    model = model or DummyModel()
    env = BuildEnv(torch.float32, torch.device("cpu"), EmulatedKernels())
    return InferenceEngine(model, cfg, env, allocate=False), model


def all_released(engine):
    engine.cache.check_invariants()
    return all(int(g.pool.ref_counts.sum()) == 0 for g in engine.cache.groups) and engine.cache.n_free_slots == engine.config.max_seqs


def test_release_on_finish_and_reuse_without_reset():
    # the reference's tests/inference/test_engine.py:62-112: the model always emits 3, which is the stop token
    engine, _ = make_engine()
    reqs = [Request(prompt_tokens=p, request_id=i, decode_params=SeqDecodingParams(max_num_tokens=len(p) + 5, stop_tokens=[[3]]))
            for i, p in enumerate([[7, 7], [1]])]
    res = engine.generate(reqs)
    assert res.tokens == [[3], [3]]  # generated tokens only, the stopping token included
    assert res.finish_reasons == ["stop", "stop"]
    assert all_released(engine)
    res = engine.generate(reqs)  # usable again without reset()
    assert res.tokens == [[3], [3]] and all_released(engine)


def test_length_limit_counts_the_prompt():
    engine, _ = make_engine()
    r = Request(prompt_tokens=[1, 2, 4], request_id=0, decode_params=SeqDecodingParams(max_num_tokens=7))
    res = engine.generate([r])
    assert res.tokens == [[3, 3, 3, 3]] and res.finish_reasons == ["length"] and res.total_generated == 4
    res = engine.generate([Request(prompt_tokens=[1, 2, 4], request_id=1, max_new_tokens=2)])
    assert res.tokens == [[3, 3]]


def test_stop_sequence_may_begin_in_the_prompt():
    engine, _ = make_engine(DummyModel(count=True))
    # counts 5, 6, 7 ...; the stop sequence [4, 5] straddles the end of the prompt
    res = engine.generate([Request(prompt_tokens=[2, 4], request_id=0, max_new_tokens=6, stop_tokens=[[4, 5]])])
    assert res.tokens == [[5]]
    res = engine.generate([Request(prompt_tokens=[2, 4], request_id=0, max_new_tokens=6, stop_tokens=[[9, 9], [6, 7]])])
    assert res.tokens == [[5, 6, 7]]


def test_stop_signal_reference_vectors():
    # tests/inference/test_inference_utils.py:9-88
    assert is_stop_signal([5, 6, 7], [[5, 6, 7]])
    assert not is_stop_signal([5, 6, 7], [[1, 2, 3]])
    assert is_stop_signal([5, 6, 7], [[6, 7]])
    assert not is_stop_signal([1, 2, 3], [])
    assert not is_stop_signal([1, 2, 3], [[]])
    assert is_stop_signal([8, 9, 10], [[1, 2, 3], [8, 9, 10], [4, 5, 6]])
    assert not is_stop_signal([28070, 5573, 323, 8254, 1667, 4227, 11, 1057, 2291, 69, 19568, 323, 40317, 743, 704], [[13]])


def test_more_requests_than_slots_and_order_of_results():
    engine, model = make_engine(DummyModel(count=True), max_seqs=2)
    reqs = [Request(prompt_tokens=[i], request_id=i, max_new_tokens=3) for i in range(5)]
    res = engine.generate(reqs)
    assert res.tokens == [[(i + 1) % 10, (i + 2) % 10, (i + 3) % 10] for i in range(5)]
    assert all_released(engine)
    assert max(len(b) for b in model.batches) <= 2  # never more than two live sequences


def test_prompts_are_cut_under_the_token_budget_and_mixed_with_decoding():
    engine, model = make_engine(DummyModel(vocab_size=100, count=True), max_prefill_size=7, max_pages_per_seq=8)
    reqs = [Request(prompt_tokens=list(range(1, 1 + n)), request_id=i, max_new_tokens=4) for i, n in enumerate([3, 20, 9])]
    res = engine.generate(reqs)
    assert [len(t) for t in res.tokens] == [4, 4, 4]
    assert res.tokens[1] == [21, 22, 23, 24]
    for b in model.batches:  # a step never holds more than 7 prompt tokens
        assert sum(n for n in b if n > 1) <= 7
    # some step holds a portion of a prompt beside a single decoded token
    assert any(1 in b and any(n > 1 for n in b) for b in model.batches)
    # the 20-token prompt went in as portions
    assert any(1 < n < 20 for b in model.batches for n in b)
    assert all_released(engine)


def test_pages_run_out_preempts_the_youngest_and_recomputes():
    # 6 pages of 16 tokens per group; two requests of 40 + 40 tokens need 3 pages each at the end, but a third
    # one arrives: somebody has to give way, and the tokens equal an unconstrained run
    big, _ = make_engine(DummyModel(count=True), max_pages=64, max_pages_per_seq=8)
    small, model = make_engine(DummyModel(count=True), max_pages=6, max_pages_per_seq=8)
    reqs = [Request(prompt_tokens=[i] * 30, request_id=i, max_new_tokens=30) for i in range(3)]
    want = big.generate(reqs)
    got = small.generate(reqs)
    assert small.scheduler.n_preemptions > 0
    assert got.tokens == want.tokens
    assert got.finish_reasons == ["length"] * 3
    assert all_released(small)


def test_a_request_too_large_for_the_pool_fails_alone():
    engine, _ = make_engine(DummyModel(count=True), max_pages=2, max_pages_per_seq=8)
    reqs = [Request(prompt_tokens=[1] * 10, request_id=0, max_new_tokens=3),
            Request(prompt_tokens=[2] * 40, request_id=1, max_new_tokens=3),
            Request(prompt_tokens=[3] * 10, request_id=2, max_new_tokens=3)]
    res = engine.generate(reqs)
    assert res.finish_reasons[0] == "length" and res.finish_reasons[2] == "length"
    assert res.finish_reasons[1].startswith("error: out of pages")
    assert res.tokens[0] == [2, 3, 4] and res.tokens[2] == [4, 5, 6]
    assert all_released(engine)


def test_request_validation():
    engine, _ = make_engine(DummyModel(max_positions=32))
    with pytest.raises(ValueError, match="empty prompt"):
        engine.generate([Request(prompt_tokens=[], request_id=0, max_new_tokens=1)])
    with pytest.raises(ValueError, match="outside the vocabulary"):
        engine.generate([Request(prompt_tokens=[10], request_id=0, max_new_tokens=1)])
    with pytest.raises(ValueError, match="n_generations"):
        engine.generate([Request(prompt_tokens=[1], request_id=0, max_new_tokens=1, n_generations=9)])
    with pytest.raises(ValueError, match="longer than the limit"):
        engine.generate([Request(prompt_tokens=[1] * 33, request_id=0, max_new_tokens=1)])
    # a prompt that fills the positions exactly still yields the one token its last logits give
    res = engine.generate([Request(prompt_tokens=[1] * 32, request_id=0, max_new_tokens=5)])
    assert res.tokens == [[3]] and res.finish_reasons == ["length"]
    with pytest.raises(ValueError, match="stop sequences"):
        engine.generate([Request(prompt_tokens=[1], request_id=0, max_new_tokens=1, stop_tokens=[[1]] * 5)])
    with pytest.raises(ValueError, match="logprobs"):
        engine.generate([Request(prompt_tokens=[1], request_id=0, max_new_tokens=1, enable_logprobs=True)])
    # the model's positions bound the length: generation stops at 32 tokens in all
    res = engine.generate([Request(prompt_tokens=[1] * 30, request_id=0, max_new_tokens=10)])
    assert len(res.tokens[0]) == 2 and res.finish_reasons == ["length"]


def test_n_generations_and_logprobs_and_reset():
    engine, _ = make_engine(enable_logprobs=True)
    r = Request(prompt_tokens=[1, 2], request_id=0, max_new_tokens=2, n_generations=3, enable_logprobs=True)
    res = engine.generate([r])
    assert res.tokens == [[3, 3]] * 3
    lp = float(torch.log_softmax(torch.tensor([0.0] * 3 + [1.0] + [0.0] * 6), -1)[3])
    assert all(abs(x - lp) < 1e-6 for row in res.logprobs for x in row)
    engine.enqueue_requests([r])
    engine.step()
    assert not all_released(engine)
    engine.reset()
    assert all_released(engine)


def test_temperature_sampling_depends_on_request_and_position_only():
    # the same request gives the same tokens alone and among others, whatever the budget
    def run(reqs, **kw):
        engine, _ = make_engine(DummyModel(vocab_size=50), **kw)
        return engine.generate(reqs)

    mine = Request(prompt_tokens=[1, 2, 3, 4, 5, 6, 7, 8, 9], request_id=7, max_new_tokens=12, temperature=5.0)
    alone = run([mine]).tokens[0]
    others = [Request(prompt_tokens=[4] * n, request_id=i, max_new_tokens=9, temperature=3.0) for i, n in enumerate([1, 20, 5])]
    mixed = run(others + [mine], max_prefill_size=7).tokens[3]
    assert alone == mixed
    assert len(set(alone)) > 3  # it is sampling, not the argmax
    again = run([Request(prompt_tokens=mine.prompt_tokens, request_id=8, max_new_tokens=12, temperature=5.0)]).tokens[0]
    assert again != alone  # another request id, another key


def test_steps_launched_ahead_change_nothing():
    """Decode steps are launched before the tokens of the step before are read back. The same requests with and
    without that: the same tokens, reasons and log-probabilities, although a stop sequence ends requests after a
    step with them has been launched already, requests end by length at different times (the rows of the step
    launched ahead are then a selection of the rows before), and a request arrives while others decode."""
    def run(lookahead):
        engine, model = make_engine(DummyModel(vocab_size=40, count=True), decode_lookahead=lookahead, enable_logprobs=True, max_seqs=8)
        reqs = [Request(prompt_tokens=[1, 2, 3], request_id=0, decode_params=SeqDecodingParams(max_num_tokens=30, stop_tokens=[[9, 10]]), enable_logprobs=True),
                Request(prompt_tokens=[20], request_id=1, max_new_tokens=5, enable_logprobs=True),
                Request(prompt_tokens=[5, 6], request_id=2, max_new_tokens=12, temperature=0.9, enable_logprobs=True),
                Request(prompt_tokens=[30, 31, 32, 33], request_id=3, decode_params=SeqDecodingParams(max_num_tokens=25, stop_tokens=[[38]]))]
        seqs = engine.enqueue_requests(reqs[:3])
        for _ in range(4):
            engine.step()
        seqs += engine.enqueue_requests(reqs[3:])  # arrives while a step launched ahead is under way
        while not all(s.done for s in seqs):
            engine.step()
        assert engine._pending is None and all_released(engine)
        return [(list(s.generated), s.finish_reason, [round(x, 5) for x in s.logprobs]) for s in seqs], model.batches

    with_la, batches_la = run(True)
    without, batches = run(False)
    assert with_la == without
    assert with_la[0][0][-2:] == [9, 10] and with_la[0][1] == "stop" and with_la[1][1] == "length"
    # a step launched ahead carried one row too many whenever a stop sequence ended a request: more rows in all, never fewer steps
    assert sum(map(sum, batches_la)) > sum(map(sum, batches)) and len(batches_la) >= len(batches)


@pytest.mark.parametrize("seed", range(6))
def test_steps_with_prompt_portions_and_admissions_are_launched_ahead_too(seed):
    """Random requests arriving over time, prompts cut into small portions, few slots and pages: with steps launched
    ahead (prompt portions and admissions included) every request generates what it generates without, nothing is
    lost from the pools, and steps really were launched before their predecessor's tokens were read."""
    import random

    rng = random.Random(seed)
    n = 14
    reqs = []
    for i in range(n):
        new = rng.choice([1, 2, 6, 15])
        plen = rng.choice([1, 2, 5, 17, 33, 40])
        stop = [[rng.randrange(40)], [rng.randrange(40), rng.randrange(40)]] if rng.random() < 0.5 else None
        reqs.append(dict(prompt_tokens=[rng.randrange(40) for _ in range(plen)], request_id=i, enable_logprobs=True,
                         decode_params=SeqDecodingParams(max_num_tokens=plen + new, stop_tokens=stop, temperature=rng.choice([0.0, 0.8]))))
    arrivals = sorted(rng.randrange(0, 30) for _ in range(n)) + [10 ** 9]
    kw = dict(max_pages=rng.choice([12, 20, 64]), max_seqs=rng.choice([3, 5, 8]), max_prefill_size=rng.choice([5, 16, 64]),
              max_seqs_in_prefill=rng.choice([1, 4]), enable_logprobs=True)

    def run(lookahead):
        engine, model = make_engine(DummyModel(vocab_size=40, count=True), decode_lookahead=lookahead, **kw)
        seqs, pending, step, ahead = [], [Request(**r) for r in reqs], 0, 0
        while pending or not all(s.done for s in seqs):
            while pending and arrivals[len(seqs)] <= step:
                seqs += engine.enqueue_requests([pending.pop(0)])
            engine.step()
            ahead += engine._pending is not None
            step += 1
            assert step < 5000
        assert engine._pending is None and all_released(engine)
        return [(list(s.generated), s.finish_reason, [round(x, 5) for x in s.logprobs]) for s in seqs], ahead, model.batches

    with_la, ahead, batches_la = run(True)
    without, none_ahead, _ = run(False)
    assert with_la == without
    assert none_ahead == 0 and ahead > 0
    assert any(max(b) > 1 and len(b) > 1 for b in batches_la)  # portions of prompts beside decoded tokens in one step


@pytest.mark.parametrize("lookahead", [True, False])
def test_a_lone_request_that_runs_out_of_pages_while_decoding_ends_with_its_own_error(lookahead):
    # 2 pages of 16 tokens: a prompt of 10 tokens decodes until position 32 would need a third page
    engine, _ = make_engine(DummyModel(vocab_size=50, count=True), max_pages=2, max_pages_per_seq=8, decode_lookahead=lookahead)
    other = Request(prompt_tokens=[7], request_id=1, max_new_tokens=2)
    res = engine.generate([Request(prompt_tokens=[1] * 10, request_id=0, max_new_tokens=40), other])
    assert res.finish_reasons[0].startswith("error: out of pages")
    # tokens 10 .. 31 are in the cache (22 generated ones were fed back) and the 23rd was sampled from the last step
    assert res.tokens[0] == [(2 + i) % 50 for i in range(len(res.tokens[0]))] and len(res.tokens[0]) in (22, 23)
    assert res.finish_reasons[1] == "length" and res.tokens[1] == [8, 9]  # the other request's result is not lost
    assert all_released(engine)


@pytest.mark.parametrize("lookahead", [True, False])
def test_fewer_tokens_a_round_than_decoding_requests_take_turns(lookahead):
    """``max_tokens_per_round`` below the number of decoding requests: nobody waits for the older ones to end."""
    engine, model = make_engine(DummyModel(vocab_size=100, count=True), max_tokens_per_round=2, decode_lookahead=lookahead)
    reqs = [Request(prompt_tokens=[10 * i + 1], request_id=i, max_new_tokens=6) for i in range(4)]
    seqs = engine.enqueue_requests(reqs)
    engine.step()  # the four prompts (one token each) in one step
    progress = []
    ahead = 0
    while not all(s.done for s in seqs):
        engine.step()
        ahead += engine._pending is not None
        progress.append([len(s.generated) for s in seqs])
    for a, b in zip(progress, progress[2:]):  # within any two steps every unfinished request has advanced
        assert all(y > x or y == 6 for x, y in zip(a, b)), (a, b)
    assert all(len(b) <= 2 for b in model.batches[1:])
    assert [s.generated for s in seqs] == [[10 * i + 2 + j for j in range(6)] for i in range(4)]
    assert (ahead > 0) == lookahead  # steps are still launched ahead
    assert all_released(engine)


def test_max_rounds_is_the_number_of_decode_steps_between_two_looks_at_the_queue():
    engine, model = make_engine(DummyModel(vocab_size=100, count=True), max_rounds=4, decode_lookahead=False)
    first = engine.enqueue_requests([Request(prompt_tokens=[1, 2, 3], request_id=0, max_new_tokens=30)])
    engine.step()
    engine.step()
    late = engine.enqueue_requests([Request(prompt_tokens=[50, 51], request_id=1, max_new_tokens=3)])
    n0 = len(model.batches)
    while not late[0].done:
        engine.step()
    joined = next(i for i, b in enumerate(model.batches) if len(b) == 2)
    # the queue was looked at before step 0; steps 0 .. 3 run without a look, step 4 follows the next one
    assert joined > n0 and joined == 4
    assert model.batches[joined] == [1, 2]
    assert late[0].generated == [52, 53, 54]
    engine.reset()
    assert all_released(engine)


def test_warm_up_meets_the_row_counts_of_serving():
    """Prompts up to a whole portion alone, batches of single tokens, and a whole portion beside decoding requests (their
    number of rows is what the matrix products of a mixed step see); afterwards the engine is as it was."""
    engine, model = make_engine(max_pages=4096, max_seqs=64, max_pages_per_seq=64, max_prefill_size=256, max_seqs_in_prefill=64)
    engine.warm_up(token_counts=[32, 256])
    shapes = {(len(b), sum(b)) for b in model.batches}
    assert {(1, 32), (1, 256), (64, 64), (32, 32), (2, 257)} <= shapes, sorted(shapes)
    assert engine.scheduler.idle and all_released(engine)


def test_warm_up_fills_a_step_s_budget_with_several_prompts_when_one_request_cannot_hold_it():
    """``max_prefill_size`` is a step's budget, ``page_size * max_pages_per_seq`` a request's limit: where the budget is
    larger (the 20B workload: 2,048 prompt tokens a step, requests of 1,552), serving runs steps of several prompts, and
    the ladder has to reach their row counts."""
    engine, model = make_engine(max_pages=256, max_seqs=8, max_pages_per_seq=4, max_prefill_size=150, max_seqs_in_prefill=4)
    engine.warm_up()
    sums = {sum(b) for b in model.batches}
    assert 150 in sums and 63 in sums, sorted(sums)
    assert any(sum(b) == 150 and b == [63, 63, 24] for b in model.batches)
    assert any(len(b) > 3 and sum(b) > 150 for b in model.batches), "a whole budget beside decoding requests"
    assert engine.scheduler.idle and all_released(engine)
