"""The engine on the GPU beyond replay: each part alone against its plain function, long decoding,
the first tokens of a sequence, generation through the entry point (greedy and sampled), and the
generality of the parts: a window, a layer named twice, a layer that reads another layer's cache,
and a toy mixer with state of its own that is registered here, without a change to the framework."""
import math
from dataclasses import dataclass

import pytest
import torch

import plain_gpt2 as P
from emulated_kernels import gumbel_noise
from helpers import make_meta, read_weights, toy_rotary_unit, write_model
from tiny_configs import TINY, TINY_A, TINY_B

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _env(dtype):
    from levanter_amd.engine.loading import make_env

    return make_env(dtype)


def _ctx(env, tokens, runs):
    """A StepContext without a cache, for parts that need none."""
    from levanter_amd.parts import StepContext

    t = torch.tensor(tokens, dtype=torch.int32, device=DEV)
    return StepContext(kernels=env.kernels, dtype=env.dtype, device=env.device, n_tokens=len(tokens), tokens=t,
                       attention=make_meta(runs, DEV), seq_slots=torch.zeros(len(runs), dtype=torch.int32, device=DEV),
                       host={"run_lengths": [q for q, _ in runs], "first_positions": [k - q for q, k in runs], "slots": [0] * len(runs)})


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_part_alone(name, dtype):
    from levanter_amd.config import InferenceEngineConfig, LmConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache

    raw, seed = TINY[name]
    d = write_model(raw, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    w = read_weights(d)
    env = _env(dtype)
    _, model = load_model(d, env)
    s = P.plain_sizes(raw)
    rnd = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == "float32" else dict(rtol=2e-2, atol=2e-3)
    T = 23
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, s["V"], (T,), generator=g)
    ctx = _ctx(env, toks.tolist(), [(T, T)])
    # embedding with the position encoding
    x = model.embedding(ctx)
    want_x = P.plain_embed(toks, torch.arange(T), w["wte.weight"], w["wpe.weight"])
    torch.testing.assert_close(x.cpu().double(), want_x, rtol=1e-6, atol=1e-7)
    # a shifted portion uses absolute positions
    ctx5 = _ctx(env, toks[5:].tolist(), [(T - 5, T)])
    torch.testing.assert_close(model.embedding(ctx5).cpu().double(), want_x[5:], rtol=1e-6, atol=1e-7)
    blk = model.blocks[1]
    # norm
    xin = (torch.randn(T, s["D"], generator=g) * 2 + 0.5)
    h = blk.norm1(xin.to(DEV), ctx)
    want_h = rnd(P.plain_layernorm(xin.double(), w["h.1.ln_1.weight"], w["h.1.ln_1.bias"], raw["layer_norm_epsilon"]))
    torch.testing.assert_close(h.cpu().double(), want_h, **tol)
    # feed-forward (adds to the residual in place)
    hin = rnd(torch.randn(T, s["D"], generator=g).double())
    res = torch.randn(T, s["D"], generator=g)
    xr = res.to(DEV).clone()
    blk.feed_forward.forward(hin.to(env.dtype).to(DEV), xr, ctx)
    want = res.double() + P.plain_mlp(hin, w, "h.1.", raw, rnd)
    torch.testing.assert_close(xr.cpu().double(), want, **tol)
    # head on gathered rows
    rows = torch.tensor([T - 1, 3], dtype=torch.int32, device=DEV)
    hf = model.final_norm(xin.to(DEV), ctx, rows=rows)
    logits = model.head(hf, ctx)
    want_hf = rnd(P.plain_layernorm(xin.double()[[T - 1, 3]], w["ln_f.weight"], w["ln_f.bias"], raw["layer_norm_epsilon"]))
    torch.testing.assert_close(logits.cpu().double(), want_hf @ w["wte.weight"].T, **tol)
    # the mixer, through a cache of its own: a whole sequence, then the same cut in two portions
    cfg = InferenceEngineConfig(max_pages=8, max_seqs=2, page_size=16, max_pages_per_seq=4, compute_dtype=dtype)
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    want_a = P.plain_attention_layer(hin, w, "h.1.", raw, 1, rnd)
    for cuts in ([T], [9, T - 9]):
        hnd = cache.open("x")
        got = []
        i = 0
        for n in cuts:
            cache.extend(hnd, n)
            mctx = _ctx(env, toks[i:i + n].tolist(), [(n, i + n)])
            from levanter_amd.parts import CacheUnitView, GroupView

            grp = cache.groups[0]
            bt = torch.tensor(grp.block_tables[[hnd.slot], :4], device=DEV)
            dest = torch.tensor([cache.destination(grp, hnd, p) for p in range(i, i + n)], dtype=torch.int32, device=DEV)
            k_pages, v_pages, _ = cache.unit_pages(1)
            unit = CacheUnitView(k_pages=k_pages, v_pages=v_pages, group=GroupView(16, bt, dest))
            xz = torch.zeros(n, s["D"], device=DEV)
            blk.mixer.forward(hin[i:i + n].to(env.dtype).to(DEV), xz, mctx, unit, True)
            got.append(xz.cpu().double())
            cache.advance(hnd, n)
            i += n
        torch.testing.assert_close(torch.cat(got), want_a, **tol)
        cache.close(hnd)


def _engine(d, dtype, **kw):
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine

    cfg = InferenceEngineConfig(**{**dict(max_seqs=4, page_size=16, max_pages_per_seq=16, compute_dtype=dtype), **kw})
    return InferenceEngine.from_pretrained(d, cfg)


def _check_greedy(weights, raw, prompt, generated, rounding=lambda x: x, margin=1e-4):
    """Every generated token is the plain implementation's argmax after the tokens before it (where the
    plain top two are further apart than ``margin``)."""
    toks = list(prompt) + list(generated)
    logits = P.plain_logits(weights, raw, torch.tensor(toks), rounding=rounding)
    n_clear = 0
    for i, tok in enumerate(generated):
        row = logits[len(prompt) - 1 + i]
        top = row.topk(2).values
        if float(top[0] - top[1]) > margin:
            n_clear += 1
            assert int(row.argmax()) == tok, f"generated token {i}"
    return n_clear


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype):
    # the workload of tiny configuration A: prompts of 5, 17 and 33 tokens, 16 greedy tokens each
    from levanter_amd.engine import Request

    d = write_model(TINY_A, 0, torch.float32 if dtype == "float32" else torch.bfloat16)
    w = read_weights(d)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (5, 17, 33)]
    engine = _engine(d, dtype)
    res = engine.generate([Request(prompt_tokens=p, request_id=i, max_new_tokens=16) for i, p in enumerate(prompts)])
    assert [len(t) for t in res.tokens] == [16, 16, 16] and res.finish_reasons == ["length"] * 3
    if dtype == "float32":
        for p, out in zip(prompts, res.tokens):
            assert out == P.plain_greedy_generate(w, TINY_A, p, 16)
    else:
        # 47 of the 48 tokens have a margin that clear along the plain implementation's own path
        clear = sum(_check_greedy(w, TINY_A, p, out, P.bf16_rounding, margin=2e-2) for p, out in zip(prompts, res.tokens))
        assert clear >= 45
    engine.cache.check_invariants()
    assert engine.cache.n_free_slots == 4
    # the reference's constructors from a model that is already built (src/levanter/inference/engine.py:705-759): same tokens
    from levanter_amd.engine import InferenceEngine

    again = InferenceEngine.from_model(engine.model, None, max_pages=64, max_seqs=4, page_size=16, max_pages_per_seq=8,
                                       compute_dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    assert again.generate([Request(prompt_tokens=p, request_id=i, max_new_tokens=16) for i, p in enumerate(prompts)]).tokens == res.tokens
    with pytest.raises(ValueError, match="was built in"):
        InferenceEngine.from_model(engine.model, None, max_pages=64, max_seqs=4, page_size=16, max_pages_per_seq=8,
                                   compute_dtype="float32" if dtype == "bfloat16" else "bfloat16")


def test_warm_up_leaves_the_engine_as_it_found_it():
    from levanter_amd.engine import Request

    d = write_model(TINY_A, 0, torch.float32)
    reqs = [Request(prompt_tokens=[5, 6, 7, 8], request_id=0, max_new_tokens=8, temperature=0.9, key=3)]
    cold = _engine(d, "float32", max_seqs=32).generate(reqs).tokens
    engine = _engine(d, "float32", max_seqs=32)
    engine.warm_up()
    assert engine.scheduler.idle and engine.cache.n_free_slots == 32
    engine.cache.check_invariants()
    assert all(int(g.pool.ref_counts.sum()) == 0 for g in engine.cache.groups)
    assert engine.generate(reqs).tokens == cold
    engine.enqueue_requests(reqs)
    engine.step()
    with pytest.raises(RuntimeError, match="idle"):
        engine.warm_up()


def _random_requests(rng, vocab, max_pos, n):
    from levanter_amd.engine import SeqDecodingParams

    reqs = []
    for i in range(n):
        new = rng.choice([1, 2, 7, 20, 40])
        plen = min(rng.choice([1, 2, 5, 17, 33, 64, 90]), max_pos - new - 1)
        stop = None
        if rng.random() < 0.4:
            stop = [[rng.randrange(vocab)] for _ in range(rng.choice([1, 3]))] + [[rng.randrange(vocab), rng.randrange(vocab)]]
        reqs.append(dict(prompt_tokens=[rng.randrange(vocab) for _ in range(plen)], request_id=i,
                         decode_params=SeqDecodingParams(max_num_tokens=plen + new, stop_tokens=stop,
                                                         temperature=rng.choice([0.0, 0.0, 0.7, 1.5]))))
    return reqs


def _serve(d, dtype, reqs, arrivals, poison=False, **kw):
    """Requests that arrive at given steps, through enqueue_requests and step; returns what each generated and why it ended.
    ``poison``: every page holds NaN before the first request, as a page may that another request has left behind."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine, Request

    engine = InferenceEngine.from_pretrained(d, InferenceEngineConfig(compute_dtype=dtype, page_size=16, seed=3, **kw))
    if poison:
        for g in engine.cache.groups:
            g.k_pages.fill_(float("nan"))
            g.v_pages.fill_(float("nan"))
    seqs, pending, step = [], [Request(**r) for r in reqs], 0
    while pending or not all(s.done for s in seqs):
        while pending and arrivals[len(seqs)] <= step:
            seqs += engine.enqueue_requests([pending.pop(0)])
        engine.step()
        step += 1
        assert step < 20000
    engine.cache.check_invariants()
    assert all(int(g.pool.ref_counts.sum()) == 0 for g in engine.cache.groups)
    _serve.keys = [s.key for s in seqs]  # of the last run: a request's sampling key depends on the seed and its id alone
    return [(list(s.generated), s.finish_reason) for s in seqs], engine.scheduler.n_preemptions


def _parted_at_a_near_tie(weights, raw, req, key, a, b, margin):
    """Two runs of one request gave the token lists ``a`` and ``b``: at the first place where they part, the two tokens are
    the two best candidates of the plain implementation (rounded to bfloat16 where the engine rounds), noise of the
    request's key included where it samples, and they are within ``margin`` of each other."""
    i = next((j for j, (x, y) in enumerate(zip(a, b)) if x != y), None)
    if i is None:  # one is a prefix of the other: a stop sequence or the end was met in one run only, so they parted before
        raise AssertionError("one run's tokens are a prefix of the other's")
    prompt = req["prompt_tokens"]
    temperature = req["decode_params"].temperature
    pos = len(prompt) - 1 + i
    logits = P.plain_logits(weights, raw, torch.tensor(list(prompt) + list(a[:i])), rounding=P.bf16_rounding)[pos].float()
    if temperature > 0:
        logits = logits / temperature + gumbel_noise(key[0], key[1], pos, raw["vocab_size"])
    top = logits.topk(2)
    assert {a[i], b[i]} == set(top.indices.tolist()), (i, a[i], b[i], top)
    assert float(top.values[0] - top.values[1]) < margin, (i, top)


@pytest.mark.parametrize("trial", range(4))
def test_random_arrivals_small_pools_and_preemption_change_no_token(trial):
    """Random requests (greedy and sampled, with stop sequences) arriving over time into pools so small that requests wait
    and are preempted: the tokens equal those of a run with room for everything at once, with and without steps launched
    ahead. In 32-bit every request agrees; in bfloat16 a prompt that is recomputed or cut elsewhere rounds differently, and a
    request may part from the other run where its two best candidates (of the plain implementation, noise included) nearly
    tie: that they do is checked at the first token that differs."""
    import random

    name, dtype = "AB"[trial % 2], ["float32", "bfloat16"][(trial // 2) % 2]
    raw, seed = TINY[name]
    d = write_model(raw, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    rng = random.Random(100 + trial)
    n = 12
    reqs = _random_requests(rng, raw["vocab_size"], raw["n_positions"], n)
    arrivals = sorted(rng.randrange(0, 40) for _ in range(n)) + [10 ** 9]
    small = dict(max_pages=rng.choice([10, 14]), max_seqs=rng.choice([3, 4, 8]), max_pages_per_seq=8, max_prefill_size=rng.choice([7, 32]))
    ahead, _ = _serve(d, dtype, reqs, arrivals, decode_lookahead=True, **small)
    plain, _ = _serve(d, dtype, reqs, arrivals, decode_lookahead=False, poison=True, **small)  # what a page held before is never read
    roomy, n_pre = _serve(d, dtype, reqs, [0] * n + [10 ** 9], decode_lookahead=True, max_pages=200, max_seqs=32, max_pages_per_seq=8,
                          max_prefill_size=128)
    keys = _serve.keys
    assert n_pre == 0
    assert ahead == plain
    if dtype == "float32":
        assert ahead == roomy
    else:  # where a request's tokens part, its two best candidates were within rounding of each other
        w = read_weights(d)
        for i, (x, y) in enumerate(zip(ahead, roomy)):
            if x != y:
                _parted_at_a_near_tie(w, raw, reqs[i], keys[i], x[0], y[0], margin=5e-2)


def test_sampled_generation_mixed_batch_fixed_seed():
    # the workload of tiny configuration B: prompts of 1, 9, 40 and 100 tokens, prefilled in portions of 7
    # beside decoding requests, then 24 steps at temperature 0.8 with a fixed seed. Every sampled token is
    # argmax(plain logits / T + the documented noise of (request key, position)).
    from levanter_amd.engine import Request

    d = write_model(TINY_B, 1, torch.float32)
    w = read_weights(d)
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 1000, (n,), generator=g).tolist() for n in (1, 9, 40, 100)]
    engine = _engine(d, "float32", max_prefill_size=7, seed=5, enable_logprobs=True)
    reqs = [Request(prompt_tokens=p, request_id=i, max_new_tokens=24, temperature=0.8, enable_logprobs=True) for i, p in enumerate(prompts)]
    seqs = engine.enqueue_requests(reqs)
    while not all(s.done for s in seqs):
        engine.step()
    for s in seqs:
        toks = s.tokens
        logits = P.plain_logits(w, TINY_B, torch.tensor(toks))
        for i, tok in enumerate(s.generated):
            pos = s.request.prompt_tokens.__len__() - 1 + i
            scaled = logits[pos].float() / 0.8
            noisy = scaled + gumbel_noise(s.key[0], s.key[1], pos, 1000)
            top = noisy.topk(2).values
            if float(top[0] - top[1]) > 1e-3:
                assert int(noisy.argmax()) == tok
            assert abs(s.logprobs[i] - float(torch.log_softmax(scaled, -1)[tok])) < 1e-3
    # alone, the longest request gives the same tokens: sampling does not depend on the batch
    alone = _engine(d, "float32", seed=5, enable_logprobs=True).generate([reqs[3]]).tokens[0]
    assert alone == seqs[3].generated


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(dtype):
    from levanter_amd.engine import Request

    d = write_model(TINY_B, 1, torch.float32 if dtype == "float32" else torch.bfloat16)
    w = read_weights(d)
    # sharpen attention so that a wrong or stale key would change the argmax: scale the q and k columns
    # of every layer (the file is rewritten; the plain implementation reads the same file)
    from levanter_amd.weights import save_file
    from safetensors.torch import load_file
    import os

    t = load_file(os.path.join(d, "model.safetensors"))
    for i in range(3):
        t[f"h.{i}.attn.c_attn.weight"][:, :192] *= 12.0
    save_file(t, os.path.join(d, "model.safetensors"))
    w = read_weights(d)
    engine = _engine(d, dtype, max_pages=40)
    rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    margin = 1e-4 if dtype == "float32" else 3e-2
    # one prompt token, then 250 decoded tokens up to the end of the position table (256)
    res = engine.generate([Request(prompt_tokens=[7], request_id=0, max_new_tokens=400)])
    out = res.tokens[0]
    assert len(out) == 255 and res.finish_reasons == ["length"]
    # positions whose two best candidates are clearly apart (each of them is checked): 254 of 255 in bfloat16 as well
    assert _check_greedy(w, TINY_B, [7], out, rounding, margin) >= (250 if dtype == "float32" else 245)
    # the first tokens: sequences of one, two and three tokens in one batch
    res = engine.generate([Request(prompt_tokens=[5], request_id=1, max_new_tokens=3),
                           Request(prompt_tokens=[9, 4], request_id=2, max_new_tokens=2),
                           Request(prompt_tokens=[1, 2, 3], request_id=3, max_new_tokens=1)])
    for p, o in zip(([5], [9, 4], [1, 2, 3]), res.tokens):
        _check_greedy(w, TINY_B, p, o, rounding, margin)


# ------------------------------------------------------------------------------------------------
# Generality of the parts, shown with toy architectures that exist only in this test.

def _toy_spec(window=None, plan=None, n_layer=2, mixers=None):
    """A two-layer GPT-2-like description over tiny A's tensors, with options GPT-2 itself does not have."""
    from levanter_amd.config import LmConfig
    from levanter_amd.parts.spec import PlanEntry

    spec = LmConfig.from_dict(dict(TINY_A, n_layer=n_layer)).model_spec()
    for i, layer in enumerate(spec.layers):
        if window is not None and i == 1:
            layer.mixer.params["window"] = window
        if mixers and mixers[i] is not None:
            layer.mixer = mixers[i]
    if plan is not None:
        spec.plan = [PlanEntry(*p) for p in plan]
    return spec


def _run_cut(spec, tensors, dtype, toks, cuts, n_pages=16, state_checks=None):
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import make_cache
    from levanter_amd.parts import DecoderLm

    env = _env(dtype)
    model = DecoderLm(spec, tensors, env)
    cfg = InferenceEngineConfig(max_pages=n_pages, max_seqs=2, page_size=16, max_pages_per_seq=8, compute_dtype=dtype)
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    h = cache.open("t")
    out, i = [], 0
    for n in cuts:
        out.append(runner.step([StepEntry(h, toks[i:i + n], list(range(n)))]).cpu())
        cache.check_invariants()
        i += n
    return torch.cat(out), cache, h


def _plain_logits_with_a_window_in_layer_1(w, toks, W, rounding=lambda x: x):
    """Tiny A with a window of W keys in its second layer: layer 0 sees everything."""
    n = len(toks)
    x = P.plain_embed(torch.tensor(toks), torch.arange(n), w["wte.weight"], w["wpe.weight"])
    for i in range(2):
        p = f"h.{i}."
        hh = rounding(P.plain_layernorm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], 1e-5))
        q, k, v = P.plain_split_qkv(rounding(P.plain_linear(hh, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"])), 4)
        o = rounding(P.plain_causal_attention(q, k, v, window=W if i == 1 else None, rounding=rounding))
        x = x + P.plain_linear(o.transpose(0, 1).reshape(n, -1), w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
        x = x + P.plain_mlp(rounding(P.plain_layernorm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], 1e-5)), w, p, TINY_A, rounding)
    return rounding(P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5)) @ w["wte.weight"].T


def test_window_layer_has_its_own_pages_and_gives_them_back():
    d = write_model(TINY_A, 0, torch.float32)
    w = read_weights(d)
    t32 = {k: v.float() for k, v in w.items()}
    W = 20
    spec = _toy_spec(window=W)
    toks = torch.randint(0, 512, (100,), generator=torch.Generator().manual_seed(3)).tolist()
    want = _plain_logits_with_a_window_in_layer_1(w, toks, W)
    for cuts in ([100], [37, 2, 30, 1, 1, 1, 28], [1] * 100):
        got, cache, h = _run_cut(spec, t32, "float32", toks, cuts, n_pages=7)
        torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
        assert len(cache.groups) == 2
        g_all, g_win = cache.groups if cache.groups[0].requirement.window is None else cache.groups[::-1]
        assert len(g_all.pages_held(h.slot)) == 7 and len(g_win.pages_held(h.slot)) <= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_layer_beside_other_requests_in_replayed_steps(dtype):
    """Six requests decode together past their windows: steps of single tokens are filled up to eight with padding
    tokens and replayed as a graph; the padding names the first request's block 0, which its window has given back
    long ago. The window group's pool is so small that pages go round. Every row against the plain implementation."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import make_cache
    from levanter_amd.parts import DecoderLm

    store = torch.float32 if dtype == "float32" else torch.bfloat16
    d = write_model(TINY_A, 0, store)
    w = read_weights(d)
    W = 20
    env = _env(dtype)
    model = DecoderLm(_toy_spec(window=W), {k: v.to(store) for k, v in w.items()}, env)
    cfg = InferenceEngineConfig(max_pages=48, max_seqs=8, page_size=16, max_pages_per_seq=8, compute_dtype=dtype, max_prefill_size=40)
    cache = make_cache(model, cfg)
    g_all, g_win = cache.groups if cache.groups[0].requirement.window is None else cache.groups[::-1]
    assert g_all.pool.n_pages == 48 and g_win.pool.n_pages == 8 * ((W + 40 + 15) // 16 + 1)  # sized by what a window can hold
    runner = ModelRunner(model, cache, env)
    assert runner.use_graphs
    gen = torch.Generator().manual_seed(9)
    lens = [100, 90, 75, 110, 64, 101]
    seqs = [torch.randint(0, 512, (n,), generator=gen).tolist() for n in lens]
    rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    want = [_plain_logits_with_a_window_in_layer_1(w, t, W, rounding) for t in seqs]
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == "float32" else dict(rtol=2e-2, atol=8e-3)
    handles = [cache.open(i) for i in range(6)]
    done = [0] * 6
    for i, h in enumerate(handles):  # prompts of 30 .. 40 tokens, two at a time
        n = 30 + 2 * i
        got = runner.step([StepEntry(h, seqs[i][:n], list(range(n)))]).cpu()
        torch.testing.assert_close(got.double(), want[i][:n], **tol)
        done[i] = n
    worst_held = 0
    while any(done[i] < lens[i] for i in range(6)):
        live = [i for i in range(6) if done[i] < lens[i]]
        got = runner.step([StepEntry(handles[i], [seqs[i][done[i]]], [0]) for i in live]).cpu()
        for r, i in enumerate(live):
            torch.testing.assert_close(got[r].double(), want[i][done[i]], **tol, msg=lambda m: f"request {i} position {done[i]}: {m}")
            done[i] += 1
        cache.check_invariants()
        worst_held = max(worst_held, max(len(g_win.pages_held(h.slot)) for h in handles))
    assert worst_held <= 3 and g_win.block_tables[handles[0].slot, 0] == -1
    assert any(not isinstance(v, str) for v in runner._graphs.values())  # steps were replayed from a recorded graph


def test_a_layer_named_twice_and_a_layer_reading_anothers_cache():
    d = write_model(TINY_A, 0, torch.float32)
    w = read_weights(d)
    t32 = {k: v.float() for k, v in w.items()}
    toks = torch.randint(0, 512, (40,), generator=torch.Generator().manual_seed(4)).tolist()

    def plain(order):
        x = P.plain_embed(torch.tensor(toks), torch.arange(40), w["wte.weight"], w["wpe.weight"])
        kv = {}
        for layer, unit, writes in order:
            p = f"h.{layer}."
            hh = P.plain_layernorm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], 1e-5)
            q, k, v = P.plain_split_qkv(P.plain_linear(hh, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"]), 4)
            if writes:
                kv[unit] = (k, v)
            k, v = kv[unit]
            o = P.plain_causal_attention(q, k, v)
            x = x + P.plain_linear(o.transpose(0, 1).reshape(40, -1), w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
            x = x + P.plain_mlp(P.plain_layernorm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], 1e-5), w, p, TINY_A)
        return P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5) @ w["wte.weight"].T

    # layer 0 runs twice (two cache units of its own), then layer 1 reads the keys and values that the
    # first run of layer 0 wrote (unit 0) instead of writing its own
    order = [(0, 0, True), (0, 1, True), (1, 0, False)]
    want = plain(order)
    for cuts in ([40], [13, 2, 24, 1]):
        got, cache, _ = _run_cut(_toy_spec(plan=order), t32, "float32", toks, cuts)
        torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
        assert sorted(u for g in cache.groups for u in g.units) == [0, 1]
    from levanter_amd.parts import DecoderLm

    with pytest.raises(ValueError, match="before any entry has written"):
        DecoderLm(_toy_spec(plan=[(0, 0, False), (1, 1, True)]), t32, _env("float32"))


def test_a_toy_mixer_with_state_of_its_own_registers_builds_and_steps():
    """A mixer defined here: the running mean of its inputs over the request so far, kept as a sum and a
    count in a per-request slot. Registered, built from a description and stepped in portions, with the
    attention layer beside it, without touching the framework's files."""
    from levanter_amd.cache import SlotState
    from levanter_amd.parts import MIXERS, Mixer, PartSpec

    D = 64

    @MIXERS.register("toy_running_mean")
    class RunningMean(Mixer):
        def __init__(self, spec, tensors, env):
            super().__init__(spec, tensors, env)
            self.gain = float(spec.params["gain"])

        def cache_requirement(self):
            return SlotState((D + 1,), "float32")

        def forward(self, h, x, ctx, unit, writes_cache):
            t0 = 0
            for n, slot in zip(ctx.host["run_lengths"], ctx.host["slots"]):
                st = unit.state[slot]
                run = h[t0:t0 + n].float()
                sums = st[:D] + torch.cumsum(run, 0)
                counts = st[D] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)
                x[t0:t0 + n] += self.gain * sums / counts[:, None]
                st[:D] = sums[-1]
                st[D] = counts[-1]
                t0 += n

    try:
        d = write_model(TINY_A, 0, torch.float32)
        w = read_weights(d)
        t32 = {k: v.float() for k, v in w.items()}
        spec = _toy_spec(mixers=[None, PartSpec("toy_running_mean", {"gain": 0.5}, {})])
        toks = torch.randint(0, 512, (50,), generator=torch.Generator().manual_seed(6)).tolist()
        x = P.plain_embed(torch.tensor(toks), torch.arange(50), w["wte.weight"], w["wpe.weight"])
        x = P.plain_block(x, w, TINY_A, 0)
        hh = P.plain_layernorm(x, w["h.1.ln_1.weight"], w["h.1.ln_1.bias"], 1e-5)
        x = x + 0.5 * torch.cumsum(hh, 0) / torch.arange(1, 51).unsqueeze(1)
        x = x + P.plain_mlp(P.plain_layernorm(x, w["h.1.ln_2.weight"], w["h.1.ln_2.bias"], 1e-5), w, "h.1.", TINY_A)
        want = P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5) @ w["wte.weight"].T
        for cuts in ([50], [20, 2, 27, 1]):
            got, cache, h = _run_cut(spec, t32, "float32", toks, cuts)
            torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-4)
            assert list(cache.state.tensors) == [1] and float(cache.state.tensors[1][h.slot, D]) == 50.0
            cache.close(h)
            h2 = cache.open("again")  # the slot is zeroed for the next request
            assert h2.slot == h.slot and float(cache.state.tensors[1][h2.slot].abs().sum()) == 0.0
    finally:
        MIXERS.unregister("toy_running_mean")


def test_a_new_architecture_registers_without_touching_the_framework(tmp_path):
    """A configuration class and description registered under a new model_type: the folder's config.json
    picks it, the loader checks its tensors, the engine runs it."""
    import json

    from levanter_amd.config import LmConfig
    from levanter_amd.engine import InferenceEngine, Request
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.weights import write_random_model

    @LmConfig.register_subclass("toy_gpt_rms")
    @dataclass(frozen=True)
    class ToyConfig(LmConfig):
        vocab_size: int = 300
        dim: int = 48
        heads: int = 3
        layers: int = 2

        @classmethod
        def from_hf_config(cls, raw):
            return cls(**{k: raw[k] for k in ("vocab_size", "dim", "heads", "layers") if k in raw})

        def to_hf_config(self):
            return {"model_type": "toy_gpt_rms", "vocab_size": self.vocab_size, "dim": self.dim, "heads": self.heads, "layers": self.layers}

        def model_spec(self):
            from levanter_amd.config import Gpt2Config

            spec = Gpt2Config(vocab_size=self.vocab_size, n_positions=64, n_embd=self.dim, n_layer=self.layers, n_head=self.heads).model_spec()
            spec.architecture = "toy_gpt_rms"
            for layer in spec.layers:
                layer.norm1.kind = layer.norm2.kind = "rmsnorm"
            spec.final_norm.kind = "rmsnorm"
            return spec

    try:
        write_random_model(ToyConfig(), 3, str(tmp_path))
        assert json.load(open(tmp_path / "config.json"))["model_type"] == "toy_gpt_rms"
        engine = InferenceEngine.from_pretrained(str(tmp_path), InferenceEngineConfig(max_seqs=2, max_pages_per_seq=4, compute_dtype="float32"))
        res = engine.generate([Request(prompt_tokens=[1, 2, 3], request_id=0, max_new_tokens=5)])
        assert len(res.tokens[0]) == 5
        # the numbers: every generated token is the argmax of a plain computation whose norms are RMS norms
        w = read_weights(str(tmp_path))
        raw = {"n_embd": 48, "n_head": 3, "n_layer": 2, "vocab_size": 300, "n_positions": 64, "activation_function": "gelu_new"}

        def rms(x, weight, bias):
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * weight + bias

        toks = [1, 2, 3] + res.tokens[0]
        x = P.plain_embed(torch.tensor(toks), torch.arange(len(toks)), w["wte.weight"], w["wpe.weight"])
        for i in range(2):
            p = f"h.{i}."
            x = x + P.plain_attention_layer(rms(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"]), w, p, raw, i)
            x = x + P.plain_mlp(rms(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"]), w, p, raw)
        logits = rms(x, w["ln_f.weight"], w["ln_f.bias"]) @ w["wte.weight"].T
        assert logits[2:-1].argmax(-1).tolist() == res.tokens[0]
        with_layernorm = P.plain_logits(w, raw, torch.tensor(toks))
        assert float((with_layernorm - logits).abs().max()) > 1e-2  # the two norms are told apart
        step_logits = engine.runner.step([__import__("levanter_amd.engine", fromlist=["StepEntry"]).StepEntry(engine.cache.open("z"), toks, list(range(len(toks))))])
        torch.testing.assert_close(step_logits.cpu().double(), logits, rtol=1e-4, atol=1e-5)
    finally:
        LmConfig.unregister("toy_gpt_rms")


def test_other_blocks_and_another_embedding_register_without_touching_the_framework():
    """Arrangements GPT-2 does not have, defined here: a block whose mixer and feed-forward read the same normed input
    and add to the residual side by side (three parts: one norm), a block with a norm after each branch as well (six
    parts), a layer that has a mixer and no feed-forward, and an embedding that scales the token rows. Each is a class
    registered from this file and named in a description; the framework's files stay as they are."""
    from levanter_amd.parts import BLOCKS, EMBEDDINGS, Block, LayerSpec, PartSpec, TensorSpec
    from levanter_amd.parts.embedding import TokenEmbedding

    @BLOCKS.register("toy_parallel")
    class Parallel(Block):
        roles = ("norm", "mixer", "feed_forward")

        def forward(self, x, ctx, unit, writes_cache):
            h = self.parts["norm"](x, ctx)
            self.parts["mixer"].forward(h, x, ctx, unit, writes_cache)
            self.parts["feed_forward"].forward(h, x, ctx)

    @BLOCKS.register("toy_sandwich")
    class Sandwich(Block):
        roles = ("norm1", "mixer", "post1", "norm2", "feed_forward", "post2")

        def forward(self, x, ctx, unit, writes_cache):
            p = self.parts
            for pre, branch, post in (("norm1", "mixer", "post1"), ("norm2", "feed_forward", "post2")):
                y = torch.zeros_like(x)
                if branch == "mixer":
                    p[branch].forward(p[pre](x, ctx), y, ctx, unit, writes_cache)
                else:
                    p[branch].forward(p[pre](x, ctx), y, ctx)
                x += p[post](y, ctx).float()

    @BLOCKS.register("toy_mixer_only")
    class MixerOnly(Block):
        roles = ("norm1", "mixer")

        def forward(self, x, ctx, unit, writes_cache):
            self.parts["mixer"].forward(self.parts["norm1"](x, ctx), x, ctx, unit, writes_cache)

    @EMBEDDINGS.register("toy_scaled_embedding")
    class Scaled(TokenEmbedding):
        def __call__(self, ctx):
            x = super().__call__(ctx)  # token row + position row
            pos = self.position.embedding_table()[ctx.attention.positions.long()].float()
            return (x - pos) * float(self.spec.params["multiplier"]) + pos

    try:
        from levanter_amd.config import LmConfig

        raw = dict(TINY_A, n_layer=3)
        d = write_model(raw, 2, torch.float32)
        w = read_weights(d)
        t32 = {k: v.float() for k, v in w.items()}
        spec = LmConfig.from_dict(raw).model_spec()
        l0, l1, l2 = spec.layers
        spec.layers[0] = LayerSpec("toy_parallel", norm=l0.norm1, mixer=l0.mixer, feed_forward=l0.feed_forward)
        post = lambda name: PartSpec("layernorm", {"dim": 64, "eps": 1e-5, "bias": True},
                                     {"weight": TensorSpec(name + ".weight", (64,), init="one_plus_normal"), "bias": TensorSpec(name + ".bias", (64,))})
        spec.layers[1] = LayerSpec("toy_sandwich", norm1=l1.norm1, mixer=l1.mixer, post1=post("h.0.ln_2"), norm2=l1.norm2,
                                   feed_forward=l1.feed_forward, post2=post("ln_f"))  # tensors of the file, used a second time
        spec.layers[2] = LayerSpec("toy_mixer_only", norm1=l2.norm1, mixer=l2.mixer)
        spec.embedding.kind = "toy_scaled_embedding"
        spec.embedding.params["multiplier"] = 3.0
        assert "h.2.mlp.c_fc.weight" not in spec.all_tensors() and "h.0.ln_2.weight" in spec.all_tensors()
        toks = torch.randint(0, 512, (45,), generator=torch.Generator().manual_seed(12)).tolist()
        ln = lambda x, name: P.plain_layernorm(x, w[name + ".weight"], w[name + ".bias"], 1e-5)
        x = 3.0 * w["wte.weight"][torch.tensor(toks)] + w["wpe.weight"][:45]
        h = ln(x, "h.0.ln_1")
        x = x + P.plain_attention_layer(h, w, "h.0.", raw, 0) + P.plain_mlp(h, w, "h.0.", raw)
        x = x + ln(P.plain_attention_layer(ln(x, "h.1.ln_1"), w, "h.1.", raw, 1), "h.0.ln_2")
        x = x + ln(P.plain_mlp(ln(x, "h.1.ln_2"), w, "h.1.", raw), "ln_f")
        x = x + P.plain_attention_layer(ln(x, "h.2.ln_1"), w, "h.2.", raw, 2)
        want = ln(x, "ln_f") @ w["wte.weight"].T
        for cuts in ([45], [17, 2, 25, 1]):
            got, cache, _ = _run_cut(spec, t32, "float32", toks, cuts)
            torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
        with pytest.raises(ValueError, match="lacks feed_forward"):
            bad = LmConfig.from_dict(raw).model_spec()
            bad.layers[0] = LayerSpec("toy_parallel", norm=l0.norm1, mixer=l0.mixer)
            from levanter_amd.parts import DecoderLm
            DecoderLm(bad, t32, _env("float32"))
    finally:
        for k in ("toy_parallel", "toy_sandwich", "toy_mixer_only"):
            BLOCKS.unregister(k)
        EMBEDDINGS.unregister("toy_scaled_embedding")


def test_a_toy_state_mixer_that_steers_from_the_device_is_replayed_from_a_graph():
    """The running-mean mixer again, written with device-side facts only (``ctx.token_slots``, positions, request
    rows): it declares itself ``graph_safe``, so decode steps of a model that holds it are recorded and replayed,
    padding tokens and all; their logits equal the eager runner's."""
    from levanter_amd.cache import SlotState
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import make_cache
    from levanter_amd.parts import MIXERS, DecoderLm, Mixer, PartSpec

    D = 64

    @MIXERS.register("toy_running_mean_on_device")
    class RunningMean(Mixer):
        graph_safe = True

        def cache_requirement(self):
            return SlotState((D + 1,), "float32")

        def forward(self, h, x, ctx, unit, writes_cache):
            pos, seq, slots = ctx.attention.positions, ctx.attention.token_seq, ctx.token_slots
            valid = slots >= 0
            slot = slots.clamp(min=0).long()
            earlier = (seq[:, None] == seq[None, :]) & (pos[None, :] <= pos[:, None]) & valid[None, :] & valid[:, None]
            hf = h.float()
            sums = unit.state[slot, :D] + earlier.float() @ hf
            x += 0.5 * sums / (pos + 1).float()[:, None]
            unit.state.index_add_(0, slot, torch.cat([hf, torch.ones_like(hf[:, :1])], 1) * valid[:, None].float())

    try:
        d = write_model(TINY_A, 0, torch.float32)
        w = read_weights(d)
        t32 = {k: v.float() for k, v in w.items()}
        spec = _toy_spec(mixers=[None, PartSpec("toy_running_mean_on_device", {}, {})])
        env = _env("float32")
        model = DecoderLm(spec, t32, env)
        assert model.graph_safe
        cfg = InferenceEngineConfig(max_pages=32, max_seqs=8, page_size=16, max_pages_per_seq=8, compute_dtype="float32")
        gen = torch.Generator().manual_seed(14)
        seqs = [torch.randint(0, 512, (n,), generator=gen).tolist() for n in (50, 40, 45, 38, 47)]

        def plain(toks):
            n = len(toks)
            x = P.plain_embed(torch.tensor(toks), torch.arange(n), w["wte.weight"], w["wpe.weight"])
            x = P.plain_block(x, w, TINY_A, 0)
            hh = P.plain_layernorm(x, w["h.1.ln_1.weight"], w["h.1.ln_1.bias"], 1e-5)
            x = x + 0.5 * torch.cumsum(hh, 0) / torch.arange(1, n + 1).unsqueeze(1)
            x = x + P.plain_mlp(P.plain_layernorm(x, w["h.1.ln_2.weight"], w["h.1.ln_2.bias"], 1e-5), w, "h.1.", TINY_A)
            return P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5) @ w["wte.weight"].T

        want = [plain(t) for t in seqs]
        cache = make_cache(model, cfg)
        runner = ModelRunner(model, cache, env)
        assert runner.use_graphs
        handles = [cache.open(i) for i in range(5)]
        got = runner.step([StepEntry(h, seqs[i][:10 + i], list(range(10 + i))) for i, h in enumerate(handles)]).cpu()
        r0 = 0
        for i in range(5):
            torch.testing.assert_close(got[r0:r0 + 10 + i].double(), want[i][:10 + i], rtol=1e-4, atol=1e-4)
            r0 += 10 + i
        for step in range(24):  # five single tokens, filled up to eight: replayed from the second step on
            got = runner.step([StepEntry(h, [seqs[i][h.length]], [0]) for i, h in enumerate(handles)]).cpu()
            for i, h in enumerate(handles):
                torch.testing.assert_close(got[i].double(), want[i][h.length - 1], rtol=1e-4, atol=1e-4)
        assert any(not isinstance(v, str) for v in runner._graphs.values())
        for i, h in enumerate(handles):
            assert float(cache.state.tensors[1][h.slot, D]) == h.length  # padding tokens were not counted
    finally:
        MIXERS.unregister("toy_running_mean_on_device")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_a_hip_graph_equal_eager_steps(dtype, monkeypatch):
    """Steps of single tokens are captured into a HIP graph the second time their shape comes. Every replay
    is compared with the same step run eagerly by a second runner, with eager work (a prompt portion of
    another request, synchronisations) between the replays, and with pages that change from step to step."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache
    import levanter_amd.engine.step as step_mod

    monkeypatch.setattr(step_mod, "GRAPH_BLOCK_BUCKET", 4)  # so that the padded table width changes while decoding
    d = write_model(TINY_B, 1, torch.float32 if dtype == "float32" else torch.bfloat16)
    env = _env(dtype)
    _, model = load_model(d, env)
    cfg = InferenceEngineConfig(max_pages=40, max_seqs=4, page_size=16, max_pages_per_seq=16, compute_dtype=dtype)
    runners = []
    for graphs in (True, False):
        cache = make_cache(model, cfg)
        runners.append((ModelRunner(model, cache, env, use_graphs=graphs), cache))
    assert runners[0][0].use_graphs and not runners[1][0].use_graphs
    g = torch.Generator().manual_seed(9)
    toks = {k: torch.randint(0, 1000, (120,), generator=g).tolist() for k in "abc"}
    handles = [{k: c.open(k) for k in "abc"} for _, c in runners]
    for (r, _), h in zip(runners, handles):
        r.step([StepEntry(h["a"], toks["a"][:20], []), StepEntry(h["b"], toks["b"][:3], [])])
    n_graph_steps = 0
    for i in range(60):
        outs = []
        for (r, _), h in zip(runners, handles):
            ia, ib = h["a"].length, h["b"].length
            outs.append(r.step([StepEntry(h["a"], [toks["a"][ia]], [0]), StepEntry(h["b"], [toks["b"][ib]], [0])]).cpu())
            if i % 7 == 3:  # eager work between the replays: a portion of a third request
                ic = h["c"].length
                r.step([StepEntry(h["c"], toks["c"][ic:ic + 5], [4])])
                torch.cuda.synchronize()
        torch.testing.assert_close(outs[0], outs[1], rtol=0, atol=0)
        n_graph_steps += 1
    graphs = [v for v in runners[0][0]._graphs.values() if v != "seen"]
    assert len(graphs) >= 2  # the block-table bucket changed at least once while decoding 60 tokens
    assert all(r.cache.groups[0].pool.n_free < 40 for r, _ in runners)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_steps_are_filled_up_to_a_few_shapes_and_replayed_from_graphs(dtype, monkeypatch):
    """Steps of prompt portions beside single tokens are filled up (ghost single tokens to a multiple of 16, room for four
    portions, empty attention tiles, full-width block tables) so that steps with the same number of prompt tokens share a
    shape and are replayed from a HIP graph from their second occurrence on. Every such step equals the same step run
    eagerly without any filling (32-bit: bit for bit), with one to three portions, requests that end, a step whose many
    wanted rows do not fit the shape (it runs as it is), and the caches agree afterwards."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache
    import levanter_amd.engine.step as step_mod

    monkeypatch.setattr(step_mod, "MIXED_DECODE_BUCKET", 4)
    d = write_model(TINY_A, 0, torch.float32 if dtype == "float32" else torch.bfloat16)
    env = _env(dtype)
    _, model = load_model(d, env)
    cfg = InferenceEngineConfig(max_pages=120, max_seqs=16, page_size=16, max_pages_per_seq=8, compute_dtype=dtype)
    runners = []
    for graphs in (True, False):
        cache = make_cache(model, cfg)
        runners.append((ModelRunner(model, cache, env, use_graphs=graphs), cache))
    g = torch.Generator().manual_seed(21)
    names = [f"r{i}" for i in range(14)]
    toks = {k: torch.randint(0, 512, (120,), generator=g).tolist() for k in names}
    handles = [{k: c.open(k) for k in names[:6]} for _, c in runners]
    for (r, _), h in zip(runners, handles):  # six requests that decode from now on
        r.step([StepEntry(h[k], toks[k][:2 + 3 * i], []) for i, k in enumerate(names[:6])])
    live = list(names[:6])
    tol = dict(rtol=0, atol=0) if dtype == "float32" else dict(rtol=2e-2, atol=8e-3)
    # 40 prompt tokens a step, cut into one to three portions of newcomers; the single tokens go 6, 6, 5 (one ends), ...
    plans = [[("r6", 40)], [("r6", 30), ("r7", 10)], [("r7", 25), ("r8", 13), ("r9", 2)], [("r8", 40)], [("r9", 38), ("r10", 2)],
             [("r10", 40)], [("r10", 20), ("r11", 20)], [("r11", 40)], [("r12", 40)], [("r12", 33), ("r13", 7)]]
    replays = 0
    for i, plan in enumerate(plans):
        if i in (2, 6):
            gone = live.pop(1)
            for (_, c), h in zip(runners, handles):
                c.close(h.pop(gone))
        outs = []
        for (r, c), h in zip(runners, handles):
            entries = [StepEntry(h[k], [toks[k][h[k].length]], [0]) for k in live]
            for k, n in plan:
                if k not in h:
                    h[k] = c.open(k)
                entries.append(StepEntry(h[k], toks[k][h[k].length:h[k].length + n], [n - 1]))
            before = sum(1 for v in r._graphs.values() if v != "seen")
            outs.append(r.step(entries).cpu())
            c.check_invariants()
        assert outs[0].shape == (len(live) + len(plan), 512)
        torch.testing.assert_close(outs[0], outs[1], **tol, msg=lambda m: f"mixed step {i}: {m}")
    graphs = {k: v for k, v in runners[0][0]._graphs.items() if v != "seen"}
    # single tokens 6 and 5 fill up to 8, 4 stays 4: two shapes of 40 prompt tokens, both recorded and replayed
    assert len(graphs) == 2 and all(k[0] - k[4] == 40 and k[4] in (4, 8) for k in graphs), list(graphs)
    # a step that wants every row of its portion does not fit the shape's wanted rows: it runs as it is, and is right
    outs = []
    for (r, c), h in zip(runners, handles):
        k = "r13"
        n = 30
        outs.append(r.step([StepEntry(h[x], [toks[x][h[x].length]], [0]) for x in live]
                           + [StepEntry(h[k], toks[k][h[k].length:h[k].length + n], list(range(n)))]).cpu())
    assert outs[0].shape == (len(live) + 30, 512)
    torch.testing.assert_close(outs[0], outs[1], **tol)
    # what the steps wrote is the same with and without filling: every live request reads all of its cache once more
    last = []
    for (r, _), h in zip(runners, handles):
        last.append(r.step([StepEntry(h[k], toks[k][h[k].length:h[k].length + 3], [2]) for k in sorted(h)]).cpu())
    torch.testing.assert_close(last[0], last[1], **tol)


def test_more_step_shapes_than_graphs_are_kept(monkeypatch):
    """At most ``MAX_GRAPHS`` shapes are remembered; one more and every recorded graph is dropped (its shape is recorded
    again when it comes twice more). With room for 3 and a block-table width that changes every 16 tokens, 110 decode
    steps of two requests cross the limit several times and still equal the same steps run eagerly, bit for bit."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache
    import levanter_amd.engine.step as step_mod

    monkeypatch.setattr(step_mod, "GRAPH_BLOCK_BUCKET", 1)
    monkeypatch.setattr(step_mod, "MAX_GRAPHS", 3)
    d = write_model(TINY_A, 0, torch.bfloat16)
    env = _env("bfloat16")
    _, model = load_model(d, env)
    cfg = InferenceEngineConfig(max_pages=24, max_seqs=4, page_size=16, max_pages_per_seq=8, compute_dtype="bfloat16")
    runners = []
    for graphs in (True, False):
        cache = make_cache(model, cfg)
        runners.append((ModelRunner(model, cache, env, use_graphs=graphs), cache))
    g = torch.Generator().manual_seed(2)
    toks = {k: torch.randint(0, 512, (128,), generator=g).tolist() for k in "ab"}
    handles = [{k: c.open(k) for k in "ab"} for _, c in runners]
    for (r, _), h in zip(runners, handles):
        r.step([StepEntry(h["a"], toks["a"][:9], []), StepEntry(h["b"], toks["b"][:2], [])])
    most, dropped, recorded_before = 0, 0, 0
    for i in range(110):
        outs = []
        for (r, _), h in zip(runners, handles):
            outs.append(r.step([StepEntry(h[k], [toks[k][h[k].length]], [0]) for k in "ab"]).cpu())
        torch.testing.assert_close(outs[0], outs[1], rtol=0, atol=0, msg=lambda m: f"decode step {i}: {m}")
        graphs = runners[0][0]._graphs
        recorded = sum(1 for v in graphs.values() if v != "seen")
        dropped += recorded < recorded_before
        recorded_before = recorded
        most = max(most, len(graphs))
    assert dropped >= 1 and most <= 4, (dropped, most)


def test_cache_sized_from_the_free_memory_of_the_device():
    """``max_pages="auto"`` with the real query: the pool takes what is free once the weights are there, less the reserve,
    capped at ``max_seqs * max_pages_per_seq``; a generation runs in it."""
    from levanter_amd.cache.sizing import GIB, group_page_bytes
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine, Request

    d = write_model(TINY_B, 1, torch.bfloat16)
    free_before, total = torch.cuda.mem_get_info(torch.device(DEV))
    # a reserve that leaves about 1 GiB: far fewer pages than the cap, so the free memory is what decides
    reserve = max(0.0, free_before / GIB - 1.0)
    cfg = InferenceEngineConfig(max_pages="auto", cache_memory_reserve_gib=reserve, max_seqs=4096, max_pages_per_seq=256,
                                page_size=16, compute_dtype="bfloat16")
    engine = InferenceEngine.from_pretrained(d, cfg)
    (group,) = engine.cache.groups
    page_bytes = group_page_bytes(group.requirement, len(group.units), 16, 2)
    n = group.pool.n_pages
    assert 256 <= n < 4096 * 256
    assert n * page_bytes <= free_before - reserve * GIB
    assert n * page_bytes >= 0.5 * GIB, "about 1 GiB was on offer"
    assert group.k_pages.shape[1] == n and group.k_pages.is_cuda
    assert group.k_pages.numel() * 2 * 2 == n * page_bytes  # keys and values, two bytes an element
    res = engine.generate([Request(prompt_tokens=[1, 2, 3, 4, 5], request_id=0, max_new_tokens=6)])
    assert len(res.tokens[0]) == 6
    # and with a reserve larger than the device there is nothing to promise
    with pytest.raises(MemoryError, match="auto"):
        InferenceEngine.from_pretrained(d, InferenceEngineConfig(max_pages="auto", cache_memory_reserve_gib=total / GIB + 1,
                                                                  compute_dtype="bfloat16"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graphed_decode_batches_are_filled_up_with_ghost_tokens(dtype):
    """Requests end one by one: 7, 6 and 5 live requests all run the graph of 8 rows, the missing ones being ghost
    tokens that are written nowhere. Every step equals the same step run eagerly without ghosts (32-bit: bit for
    bit; bfloat16: up to the rounding of another split of the key range), and the caches stay equal afterwards."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache
    from levanter_amd.engine.step import graph_batch_bucket

    assert [graph_batch_bucket(n) for n in (1, 4, 5, 8, 9, 63)] == [1, 4, 8, 8, 16, 64]
    d = write_model(TINY_A, 0, torch.float32 if dtype == "float32" else torch.bfloat16)
    env = _env(dtype)
    _, model = load_model(d, env)
    cfg = InferenceEngineConfig(max_pages=64, max_seqs=8, page_size=16, max_pages_per_seq=8, compute_dtype=dtype)
    runners = []
    for graphs in (True, False):
        cache = make_cache(model, cfg)
        runners.append((ModelRunner(model, cache, env, use_graphs=graphs), cache))
    g = torch.Generator().manual_seed(11)
    names = "abcdefg"
    toks = {k: torch.randint(0, 512, (60,), generator=g).tolist() for k in names}
    handles = [{k: c.open(k) for k in names} for _, c in runners]
    for (r, _), h in zip(runners, handles):
        r.step([StepEntry(h[k], toks[k][:3 + 2 * i], []) for i, k in enumerate(names)])
    live = list(names)
    tol = dict(rtol=0, atol=0) if dtype == "float32" else dict(rtol=2e-2, atol=8e-3)
    for i in range(30):
        if i in (10, 20):  # a request ends: the batch shrinks, the graph does not change
            gone = live.pop(2)
            for (_, c), h in zip(runners, handles):
                c.close(h[gone])
        outs = []
        for (r, _), h in zip(runners, handles):
            outs.append(r.step([StepEntry(h[k], [toks[k][h[k].length]], [0]) for k in live]).cpu())
        assert outs[0].shape == (len(live), 512)
        torch.testing.assert_close(outs[0], outs[1], **tol)
    keys = [k for k, v in runners[0][0]._graphs.items() if v != "seen"]
    assert keys and all(k[0] == 8 and k[1] == 8 for k in keys)
    # what the steps wrote is the same with and without ghosts: one more whole-prompt-like step reads it all back
    last = []
    for (r, _), h in zip(runners, handles):
        last.append(r.step([StepEntry(h[k], toks[k][h[k].length:h[k].length + 3], [2]) for k in live]).cpu())
    torch.testing.assert_close(last[0], last[1], **tol)


def test_a_toy_rotary_position_encoding_registers_and_only_distances_count():
    """Another position encoding, defined here, with a kernel of its own: queries and keys are rotated by their absolute
    position before the cache write (pairs (i, i + head_dim/2) of a head) by a HIP kernel that lies beside this test
    (``toy_rotary.hip``), is registered as a kernel unit from here and is reached through ``kernels.call``; the embedding
    adds no position. Compared with a plain whole-sequence computation; a shift of all positions changes nothing, because
    only distances count; and the part is ``graph_safe``: the single-token steps are replayed from a HIP graph."""
    from levanter_amd.kernels import KernelError
    from levanter_amd.parts import POSITION_ENCODINGS, PartSpec, PositionEncoding

    H, HD, BASE = 4, 16, 100.0
    unit = toy_rotary_unit()

    def angles(pos):  # [T, HD/2]
        inv = BASE ** (-torch.arange(HD // 2, dtype=torch.float64) / (HD // 2))
        return pos.double()[:, None] * inv[None, :]

    def plain_rotate(x, pos):  # x [T, H, HD]
        a = angles(pos)
        c, s_ = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
        x1, x2 = x[..., : HD // 2], x[..., HD // 2:]
        return torch.cat([x1 * c - x2 * s_, x2 * c + x1 * s_], -1)

    @POSITION_ENCODINGS.register("toy_rotary")
    class ToyRotary(PositionEncoding):
        graph_safe = True  # one kernel launch whose shape follows the step's sizes; positions are read from device memory

        def rotate(self, q, k, ctx):
            kern = ctx.kernels
            for t in (q, k):  # strided views into the fused projection's output: rotated in place
                kern.call(unit, "toy_rotate", kern.tensor_ptr(t), t.stride(0), kern.tensor_ptr(ctx.attention.positions), t.shape[0],
                          t.shape[1] // HD, HD, BASE, 0 if t.dtype == torch.float32 else 1, kern.stream())

    # the kernel alone against the plain rotation, both dtypes, and its own error message through the package's channel
    kern = _env("float32").kernels
    pos = torch.tensor([0, 5, 130, 7], dtype=torch.int32, device=DEV)
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        buf = torch.randn(4, 3 * H * HD, generator=torch.Generator().manual_seed(3)).to(dt).to(DEV)
        view = buf[:, H * HD: 2 * H * HD]  # a strided view, as the keys are in the fused projection's output
        want = plain_rotate(view.double().cpu().view(4, H, HD), pos.cpu()).view(4, -1)
        kern.call(unit, "toy_rotate", kern.tensor_ptr(view), view.stride(0), kern.tensor_ptr(pos), 4, H, HD, BASE, 0 if dt == torch.float32 else 1,
                  kern.stream())
        torch.testing.assert_close(view.double().cpu(), want, rtol=tol, atol=tol)
    with pytest.raises(KernelError, match="toy_rotate: bad sizes"):
        kern.call(unit, "toy_rotate", kern.tensor_ptr(buf), buf.stride(0), kern.tensor_ptr(pos), 4, H, 15, BASE, 0, kern.stream())
    with pytest.raises(KernelError, match="no entry point"):
        kern.call(unit, "toy_rotate_backwards")
    with pytest.raises(KernelError, match="unknown kernel unit"):
        kern.call("no_such_unit", "f")

    try:
        d = write_model(TINY_A, 0, torch.float32)
        w = read_weights(d)
        t32 = {k: v.float() for k, v in w.items()}
        spec = _toy_spec()
        spec.embedding.params["position"] = None  # no learned positions
        spec.max_positions = None
        for layer in spec.layers:
            layer.mixer.params["rotary"] = PartSpec("toy_rotary", {}, {})
        toks = torch.randint(0, 512, (60,), generator=torch.Generator().manual_seed(8)).tolist()

        def plain(first_pos):
            pos = torch.arange(first_pos, first_pos + 60)
            x = w["wte.weight"][torch.tensor(toks)]
            for i in range(2):
                p = f"h.{i}."
                hh = P.plain_layernorm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], 1e-5)
                q, k, v = P.plain_split_qkv(P.plain_linear(hh, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"]), H)  # [H, T, HD]
                q = plain_rotate(q.transpose(0, 1), pos).transpose(0, 1)
                k = plain_rotate(k.transpose(0, 1), pos).transpose(0, 1)
                o = P.plain_causal_attention(q, k, v)
                x = x + P.plain_linear(o.transpose(0, 1).reshape(60, -1), w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
                x = x + P.plain_mlp(P.plain_layernorm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], 1e-5), w, p, TINY_A)
            return P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5) @ w["wte.weight"].T

        want = plain(0)
        torch.testing.assert_close(plain(37), want, rtol=1e-9, atol=1e-9)  # the plain statement itself: only distances count
        for cuts in ([60], [23, 2, 30, 1, 1, 1, 1, 1]):
            got, _, _ = _run_cut(spec, t32, "float32", toks, cuts)
            torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=2e-5)
        # replayed from a graph: the model says so, and the last single-token steps of the second cutting were replays
        from levanter_amd.parts import DecoderLm

        assert DecoderLm(spec, t32, _env("float32")).graph_safe
    finally:
        POSITION_ENCODINGS.unregister("toy_rotary")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_attention_description_with_a_soft_cap_and_a_score_bias(dtype):
    """The attention part takes ``softcap`` and a ``score_bias`` tensor from its description (what
    src/levanter/layers/attention.py:361-367 applies between scaling and mask) and hands them to the kernels: tiny A with
    both in its second layer, whole and cut into portions and single tokens, against a plain whole-sequence computation."""
    from levanter_amd.parts import TensorSpec

    H, HD, CAP, L = 4, 16, 1.5, 12
    d = write_model(TINY_A, 0, torch.float32 if dtype == "float32" else torch.bfloat16)
    w = read_weights(d)
    bias = -0.4 * torch.arange(L, dtype=torch.float64)[None, :] * torch.tensor([1.0, 0.5, 0.25, 2.0], dtype=torch.float64)[:, None]
    tensors = {k: v.float() for k, v in w.items()}
    tensors["h.1.attn.score_bias"] = bias.float()
    spec = _toy_spec()
    spec.layers[1].mixer.params["softcap"] = CAP
    spec.layers[1].mixer.tensors["score_bias"] = TensorSpec("h.1.attn.score_bias", (H, L))
    toks = torch.randint(0, 512, (50,), generator=torch.Generator().manual_seed(5)).tolist()
    rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    n = len(toks)
    x = P.plain_embed(torch.tensor(toks), torch.arange(n), w["wte.weight"], w["wpe.weight"])
    for i in range(2):
        p = f"h.{i}."
        hh = rounding(P.plain_layernorm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], 1e-5))
        q, k, v = P.plain_split_qkv(rounding(P.plain_linear(hh, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"])), H)
        s = torch.einsum("htd,hsd->hts", q, k) / math.sqrt(HD)
        if i == 1:
            dist = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).clamp(0, L - 1)
            s = CAP * torch.tanh((s + bias[:, dist]) / CAP)
        s = s.masked_fill(torch.arange(n)[None, :] > torch.arange(n)[:, None], float("-inf"))
        o = rounding(torch.einsum("hts,hsd->htd", rounding(torch.softmax(s, -1)), v))
        x = x + P.plain_linear(o.transpose(0, 1).reshape(n, -1), w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
        x = x + P.plain_mlp(rounding(P.plain_layernorm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], 1e-5)), w, p, TINY_A, rounding)
    want = rounding(P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5)) @ w["wte.weight"].T
    plain_gpt2 = P.plain_logits(w, TINY_A, torch.tensor(toks))
    assert float((want - plain_gpt2).abs().max()) > 0.05, "cap and bias must matter in this test"
    run_tensors = tensors if dtype == "float32" else {k: (v if k.endswith("score_bias") else v.to(torch.bfloat16)) for k, v in tensors.items()}
    tol = dict(rtol=1e-4, atol=2e-5) if dtype == "float32" else dict(rtol=2e-2, atol=8e-3)
    for cuts in ([50], [20, 2, 19, 1, 1, 1, 1, 1, 1, 1, 1, 1]):
        got, _, _ = _run_cut(spec, run_tensors, dtype, toks, cuts)
        torch.testing.assert_close(got.double(), want, **tol)


def test_a_toy_feed_forward_with_routing_registers_builds_and_steps():
    """A feed-forward with routing, defined here: a router picks one of two experts per token (the larger of two
    32-bit router logits), each expert is a dense unit run by the framework's own GEMM on the rows sent to it.
    It steers from the host (row lists of changing length), so it is not graph-safe and the model steps eagerly."""
    from levanter_amd.parts import FEED_FORWARDS, FeedForward, PartSpec, TensorSpec
    from levanter_amd.parts.linear import Linear

    D, F = 64, 256

    @FEED_FORWARDS.register("toy_top1_experts")
    class Top1Experts(FeedForward):
        def __init__(self, spec, tensors, env):
            super().__init__(spec, tensors, env)
            self.router = tensors["router"].to(env.device, torch.float32)  # [2, D]
            self.ups = [Linear(tensors[f"up{e}.weight"], tensors[f"up{e}.bias"], "in_out", env) for e in range(2)]
            self.downs = [Linear(tensors[f"down{e}.weight"], tensors[f"down{e}.bias"], "in_out", env) for e in range(2)]

        def forward(self, h, x, ctx):
            choice = (h.float() @ self.router.T).argmax(-1)  # router logits in 32-bit
            for e in range(2):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel() == 0:
                    continue
                m = self.ups[e](h[rows].contiguous(), ctx, activation="gelu_new")
                y = torch.zeros(rows.numel(), D, dtype=torch.float32, device=h.device)
                self.downs[e](m, ctx, residual=y)
                x[rows] += y

    try:
        d = write_model(TINY_A, 0, torch.float32)
        w = read_weights(d)
        t32 = {k: v.float() for k, v in w.items()}
        g = torch.Generator().manual_seed(12)
        extra = {"h.1.moe.router": torch.randn(2, D, generator=g)}
        for e in range(2):  # expert 0 is layer 1's own dense unit, expert 1 a second one
            src = "h.1.mlp." if e == 0 else None
            extra[f"h.1.moe.up{e}.weight"] = t32["h.1.mlp.c_fc.weight"] if src else torch.randn(D, F, generator=g) * 0.05
            extra[f"h.1.moe.up{e}.bias"] = t32["h.1.mlp.c_fc.bias"] if src else torch.randn(F, generator=g) * 0.05
            extra[f"h.1.moe.down{e}.weight"] = t32["h.1.mlp.c_proj.weight"] if src else torch.randn(F, D, generator=g) * 0.05
            extra[f"h.1.moe.down{e}.bias"] = t32["h.1.mlp.c_proj.bias"] if src else torch.randn(D, generator=g) * 0.05
        tensors = dict(t32, **extra)
        spec = _toy_spec()
        names = ["router"] + [f"{n}{e}.{k}" for e in range(2) for n in ("up", "down") for k in ("weight", "bias")]
        spec.layers[1].feed_forward = PartSpec("toy_top1_experts", {},
                                               {n: TensorSpec("h.1.moe." + n, tuple(tensors["h.1.moe." + n].shape)) for n in names})
        toks = torch.randint(0, 512, (48,), generator=torch.Generator().manual_seed(13)).tolist()
        wd = {k: v.double() for k, v in tensors.items()}
        x = P.plain_embed(torch.tensor(toks), torch.arange(48), w["wte.weight"], w["wpe.weight"])
        x = P.plain_block(x, w, TINY_A, 0)
        p = "h.1."
        hh = P.plain_layernorm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], 1e-5)
        q, k, v = P.plain_split_qkv(P.plain_linear(hh, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"]), 4)
        o = P.plain_causal_attention(q, k, v)
        x = x + P.plain_linear(o.transpose(0, 1).reshape(48, -1), w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
        h2 = P.plain_layernorm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], 1e-5)
        logits_r = h2 @ wd["h.1.moe.router"].T
        choice = logits_r.argmax(-1)
        assert 5 < int(choice.sum()) < 43  # both experts get tokens
        assert float((logits_r[:, 0] - logits_r[:, 1]).abs().min()) > 1e-3  # no token on the fence between them
        act = P.plain_activation("gelu_new")
        y = torch.zeros_like(x)
        for e in range(2):
            rows = choice == e
            m = act(h2[rows] @ wd[f"h.1.moe.up{e}.weight"] + wd[f"h.1.moe.up{e}.bias"])
            y[rows] = m @ wd[f"h.1.moe.down{e}.weight"] + wd[f"h.1.moe.down{e}.bias"]
        x = x + y
        want = P.plain_layernorm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5) @ w["wte.weight"].T
        for cuts in ([48], [17, 2, 28, 1]):
            got, _, _ = _run_cut(spec, tensors, "float32", toks, cuts)
            torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=2e-5)
        from levanter_amd.parts import DecoderLm

        assert not DecoderLm(spec, tensors, _env("float32")).graph_safe
        assert DecoderLm(_toy_spec(), t32, _env("float32")).graph_safe
    finally:
        FEED_FORWARDS.unregister("toy_top1_experts")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_launched_ahead_give_the_same_generation(dtype):
    """The engine launches a decode step before the tokens of the step before are on the host (they are fed on the
    device). With and without that the generations are the same: greedy and sampled requests, a stop sequence that
    ends a request while a step with it is already under way, requests that end by length at different times."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine, Request, SeqDecodingParams

    raw, seed = TINY["B"]
    d = write_model(raw, seed, torch.float32 if dtype == "float32" else torch.bfloat16)

    def run(lookahead):
        engine = InferenceEngine.from_pretrained(d, InferenceEngineConfig(max_pages=48, max_seqs=6, page_size=16, max_pages_per_seq=8,
                                                                          compute_dtype=dtype, decode_lookahead=lookahead, seed=5))
        first = engine.generate([Request(prompt_tokens=[11, 12, 13, 14], request_id=9, max_new_tokens=12)]).tokens[0]
        stop = [first[5], first[6]]  # a stop sequence that the greedy continuation really produces
        engine.reset()
        reqs = [Request(prompt_tokens=[11, 12, 13, 14], request_id=0, decode_params=SeqDecodingParams(max_num_tokens=60, stop_tokens=[stop])),
                Request(prompt_tokens=[7], request_id=1, max_new_tokens=9),
                Request(prompt_tokens=list(range(40, 70)), request_id=2, max_new_tokens=20, temperature=0.8),
                Request(prompt_tokens=[3, 1, 4, 1, 5], request_id=3, max_new_tokens=33, temperature=1.3)]
        res = engine.generate(reqs)
        assert engine._pending is None
        engine.cache.check_invariants()
        return res.tokens, res.finish_reasons, first

    tok_a, why_a, first = run(True)
    tok_b, why_b, _ = run(False)
    assert tok_a == tok_b and why_a == why_b
    stop = first[5:7]
    n_stop = next(n for n in range(2, 13) if first[n - 2:n] == stop)  # the greedy continuation up to the stop sequence's first end
    assert why_a[0] == "stop" and tok_a[0] == first[:n_stop] and [len(t) for t in tok_a[1:]] == [9, 20, 33]
