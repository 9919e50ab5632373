"""Configurations and entry points beyond the tiny defaults, on the GPU: other page sizes, a model without biases,
the layer widths of the 7B shape, and the command line from a folder to tokens."""
import json
import os
import re
import subprocess
import sys
import tempfile
import time

import numpy as np
import pytest
import torch

import plain_gpt2 as P
import traces as TR
from helpers import read_weights, write_model
from test_gpu_replay import LENGTHS, TOL_F32, check_all_cuttings, read_step, run_trace
from tiny_configs import TINY, TINY_A, TINY_B

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("page_size", [128, 48])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes_through_trace_run(page_size, dtype):
    """128 is the reference's default page size (src/levanter/inference/engine.py:68); 48 is no power of two, which
    the matrix-core attention does not index (bfloat16 then runs the plain-arithmetic attention kernel)."""
    raw, seed = TINY["B"]
    check_all_cuttings(f"page size {page_size}", raw, seed, dtype, LENGTHS["B"], page_size=page_size)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_without_biases(dtype):
    """``use_bias: false`` (the reference's gpt2_20b configuration, config/gpt2_20b.yaml:12): no bias tensor in the
    folder, none in any norm or projection."""
    raw = dict(TINY_A, use_bias=False, n_head=2, n_inner=136, layer_norm_epsilon=1e-4)
    d = write_model(raw, 5, torch.float32)
    assert not [k for k in read_weights(d) if k.endswith(".bias")]
    check_all_cuttings("no biases", raw, 5, dtype, [70, 45, 100, 37])


def test_a_head_size_of_40_runs_in_32_bit_and_is_refused_in_bfloat16():
    """n_embd=320 with 8 heads: head size 40, a multiple of 8 and not of 16. The 32-bit path takes it (the cache keeps keys
    in chunks of 8 head dimensions); bfloat16 needs steps of 16 and says so."""
    raw = dict(TINY_A, n_embd=320, n_head=8, n_inner=None, n_positions=140)
    check_all_cuttings("head size 40", raw, 6, "float32", [70, 45, 100, 37])
    d = write_model(raw, 6, torch.bfloat16)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "bfloat16", "--out",
                        tempfile.mkdtemp(prefix="lev_trace_"), "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "head_dim=40 must be a multiple of 16" in p.stderr


@pytest.mark.parametrize("seed", [1, 7])
def test_configurations_drawn_at_random(seed):
    """Four configurations a seed, every size and option drawn at random: one to twelve heads of 16 to 128 dimensions in
    steps of 16 (in 32-bit also 8, 24, 40, 56 and 72), one to three layers, an inner width that is any multiple of 8 or
    left to the default, a vocabulary and a position table of any size, each of the reference's activation names
    (src/levanter/utils/activation.py:18-40), three values of eps, the 1/(layer + 1) factor and the biases on or off; the
    four cuttings through ``bin/trace_run``. 32-bit is held to the tolerance of the other replay tests. bfloat16 is
    compared with the plain implementation rounded at the same places, relative to the size of the logits as at the 7B
    widths: wider models have larger logits and rounding differences that grow with them (a step's r.m.s. error within
    1.5e-2 of the logits' r.m.s., its largest within 8 times that)."""
    import random

    rng = random.Random(seed)
    acts = ["relu", "silu", "swish", "gelu", "gelu_new", "quick_gelu", "tanh"]
    for ci in range(4):
        dtype = "float32" if ci % 2 == 0 else "bfloat16"
        hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128]) if dtype == "bfloat16" else rng.choice([8, 24, 40, 16, 56, 72, 128])
        nh = rng.choice([1, 2, 3, 5, 7, 12])
        raw = dict(model_type="gpt2", n_layer=rng.choice([1, 2, 3]), n_embd=hd * nh, n_head=nh,
                   n_inner=rng.choice([None, 8 * rng.randrange(3, 300)]), vocab_size=rng.randrange(300, 6000),
                   n_positions=rng.randrange(70, 330), layer_norm_epsilon=rng.choice([1e-5, 1e-6, 3e-4]),
                   activation_function=rng.choice(acts), scale_attn_by_inverse_layer_idx=rng.random() < 0.5, use_bias=rng.random() < 0.8)
        what = f"seed {seed} configuration {ci} {dtype} {json.dumps(raw)}"
        print(what, flush=True)
        d = write_model(raw, 5 + ci, torch.float32 if dtype == "float32" else torch.bfloat16)
        weights = read_weights(d)
        n_pos = raw["n_positions"]
        reqs = TR.random_requests(raw["vocab_size"], [min(n_pos, n) for n in (rng.randrange(40, 130), 45, n_pos, rng.randrange(33, 70), 64, 33)],
                                  21 + ci)
        rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
        plain = {rid: P.plain_logits(weights, raw, torch.tensor(t), rounding=rounding) for rid, t in reqs.items()}
        steps = TR.number(TR.trace_whole(reqs) + TR.trace_prefill_then_singles(reqs) + TR.trace_portions(reqs)
                          + TR.trace_mixed(reqs, seed=3 + ci))
        out = run_trace(d, dtype, steps, TR.peak_tokens(steps))
        want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
        rms = float(torch.cat([w.flatten() for w in plain.values()]).pow(2).mean().sqrt())
        for k, w in want.items():
            got = read_step(out, k, raw["vocab_size"]).double()
            if dtype == "float32":
                torch.testing.assert_close(got, w, **TOL_F32, msg=lambda m: f"{what} step {k}: {m}")
            else:
                err = (got - w).abs()
                assert float(err.pow(2).mean().sqrt()) <= 1.5e-2 * rms and float(err.max()) <= 8 * 1.5e-2 * rms, (what, k, float(err.max()), rms)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_reference_s_schedules_through_trace_run(dtype):
    """The step schedules of the reference's paged-attention tests (tests/inference/test_paged_attention.py:293-442):
    two requests filled by [[4,2],[0,1],[0,1],[2,1],[1,2],[1,1]] tokens a step, and a prefix of 1 to 3 tokens followed
    by four chunks of 1, 2, 3 or 8 tokens of both."""
    raw, seed = TINY["B"]
    d = write_model(raw, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    weights = read_weights(d)
    reqs = TR.random_requests(raw["vocab_size"], [35, 35], 21)
    rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    plain = {rid: P.plain_logits(weights, raw, torch.tensor(t), rounding=rounding) for rid, t in reqs.items()}
    steps, owner = [], {}
    schedules = [TR.REFERENCE_RAGGED_SCHEDULE] + [TR.reference_chunk_schedule(p, c) for p in TR.REFERENCE_PREFIX_SIZES
                                                  for c in TR.REFERENCE_CHUNK_SIZES]
    for i, schedule in enumerate(schedules):
        n = sum(a for a, _ in schedule)
        ids = (f"a{i}", f"b{i}")
        owner.update({ids[0]: "r0", ids[1]: "r1"})
        steps += TR.trace_two_requests(reqs["r0"][:n], reqs["r1"][:n], schedule, ids=ids)
    TR.number(steps)
    out = run_trace(d, dtype, steps, 128)
    want = TR.expected_rows(steps, lambda rid: plain[owner[rid]])
    tol = TOL_F32 if dtype == "float32" else dict(rtol=2e-2, atol=8e-3)
    for k, w in want.items():
        torch.testing.assert_close(read_step(out, k, raw["vocab_size"]).double(), w, **tol, msg=lambda m: f"step {k}: {m}")


class _LazyLogits:
    """Rows of ``hidden @ table^T`` on demand (a vocabulary of 50,257 makes all rows of a long request too many)."""

    def __init__(self, hidden, table):
        self.hidden, self.table = hidden, table

    def __getitem__(self, i):
        return self.hidden[i] @ self.table.T


def test_layer_widths_of_the_7b_shape():
    """Two layers of the 7B shape (4,096 wide, 32 heads of 128, 16,384 inner, a vocabulary of 50,257), requests of up to
    1,810 tokens, the four cuttings through ``bin/trace_run``: the 32-bit path against the plain implementation, and
    bfloat16 against the plain implementation rounded to bfloat16 at the same places. Crosses in one model what the
    tiny configurations do not reach: the tiled and the weight-streaming GEMMs at their real sizes, decode attention
    over many key ranges with the kernel that merges them, block tables that grow past a padding step while a request
    decodes, and prompts of several attention tiles."""
    raw = {"model_type": "gpt2", "n_layer": 2, "n_embd": 4096, "n_head": 32, "n_inner": 16384, "vocab_size": 50257,
           "n_positions": 2048, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    t0 = time.time()
    reqs = TR.random_requests(raw["vocab_size"], [1810, 700, 300, 130], 13)
    # the last 32 tokens of the longest request, decoded one by one, cross position 1,792 = 7 x 256
    big = [300, 2, 129, 64, 500, 17, 257, 5]
    steps = TR.number(TR.trace_whole(reqs, want=TR.want_ends) + TR.trace_prefill_then_singles(reqs, want=TR.want_ends)
                      + TR.trace_portions(reqs, sizes=big, want=TR.want_ends)
                      + TR.trace_mixed(reqs, seed=5, sizes=(2, 17, 64, 130, 260), want=TR.want_ends))
    max_tokens = TR.peak_tokens(steps)
    assert max_tokens < sum((len(t) + 63) // 64 * 64 for t in reqs.values())  # pages are used again
    for dtype in ("float32", "bfloat16"):
        d = write_model(raw, 3, torch.float32 if dtype == "float32" else torch.bfloat16)
        # Sharper attention, so that a key that is missing, stale or of another request moves the logits: with N(0, 0.02)
        # weights the scores have a deviation of 1.6 and the best of 1,800 keys a weight of a few percent; with queries
        # and keys 1.5 times larger it has a tenth or more.
        from safetensors.torch import load_file

        from levanter_amd.weights import save_file

        t = load_file(os.path.join(d, "model.safetensors"))
        for i in range(raw["n_layer"]):
            t[f"h.{i}.attn.c_attn.weight"][:, :2 * raw["n_embd"]] *= 1.5
        save_file(t, os.path.join(d, "model.safetensors"))
        del t
        weights = read_weights(d)
        print(f"7B widths {dtype}: model written in {time.time() - t0:.0f}s, {len(steps)} steps", flush=True)
        t0 = time.time()
        rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
        plain = {rid: _LazyLogits(P.plain_hidden(weights, raw, torch.tensor(t), rounding=rounding), weights["wte.weight"])
                 for rid, t in reqs.items()}
        print(f"7B widths {dtype}: plain implementation in {time.time() - t0:.0f}s", flush=True)
        t0 = time.time()
        out = run_trace(d, dtype, steps, max_tokens)
        print(f"7B widths {dtype}: replay in {time.time() - t0:.0f}s", flush=True)
        want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
        rms = float(torch.cat([w.flatten() for w in list(want.values())[:4]]).pow(2).mean().sqrt())
        # A step compares 50,257 logits a row, tens of millions in all: rounding differences are judged by their size
        # over a step (r.m.s.) and by the largest one, both relative to the r.m.s. of the logits. 32-bit: a sum of 16,384
        # products in another order differs by about 2^-24 sqrt(16384) = 8e-6 of its size, and eight products follow one
        # another: 3e-5. bfloat16, against the plain implementation that rounds at the same places: values that round to
        # the other side of a bfloat16 step differ by 2^-8, and some do after every product and norm of two layers: 1.5e-2.
        # The largest difference among so many is 5 to 6 times the r.m.s.; 8 times is allowed. A wrong key (the sharpest
        # one has a tenth of the weight) or a wrong row would show as a step whose r.m.s. is a tenth of the logits' own
        # or more.
        rel = 3e-5 if dtype == "float32" else 1.5e-2
        stats = []
        for s in steps:
            k = s["step"]
            if k in want:
                err = (read_step(out, k, raw["vocab_size"]).double() - want[k]).abs()
                stats.append((float(err.pow(2).mean().sqrt()), float(err.max()), k, s["entries"][0]["id"]))
        worst_rms, worst_max = max(stats), max(stats, key=lambda x: x[1])
        print(f"7B widths {dtype}: logits r.m.s. {rms:.3f}; worst step r.m.s. error {worst_rms[0]:.3e} (step {worst_rms[2]} {worst_rms[3]}), "
              f"largest error {worst_max[1]:.3e} (step {worst_max[2]} {worst_max[3]})", flush=True)
        assert worst_rms[0] <= rel * rms, worst_rms
        assert worst_max[1] <= 8 * rel * rms, worst_max
        t0 = time.time()


# ---- the command line ------------------------------------------------------------------------------------------------
def _sample_lm(args, timeout=300):
    p = subprocess.run([sys.executable, "-m", "levanter_amd.main.sample_lm", *args], capture_output=True, text=True, timeout=timeout,
                       cwd=ROOT)
    assert p.returncode == 0, p.stderr[-3000:]
    rounds = {}
    for m in re.finditer(r"^round (\d+) sequence (\d+) \((\d+) tokens, (\w+)\): (\[.*\])$", p.stdout, re.M):
        r, i, n, reason, toks = int(m[1]), int(m[2]), int(m[3]), m[4], json.loads(m[5])
        assert len(toks) == n
        rounds.setdefault(r, {})[i] = (toks, reason)
    return rounds, p.stdout


def _check_greedy(weights, raw, prompt, generated, rounding, margin):
    toks = list(prompt) + list(generated)
    logits = P.plain_logits(weights, raw, torch.tensor(toks), rounding=rounding)
    clear = 0
    for i, tok in enumerate(generated):
        row = logits[len(prompt) - 1 + i]
        top = row.topk(2).values
        if float(top[0] - top[1]) > margin:
            clear += 1
            assert int(row.argmax()) == tok, f"generated token {i}"
    return clear


def test_command_line_from_a_folder_to_greedy_tokens():
    """``python -m levanter_amd.main.sample_lm`` as the reference's ``sample_lm.main`` is used
    (src/levanter/main/sample_lm.py:92-195): a folder, prompts, ``max_new_tokens``, ``temperature``, ``n_rounds``; in
    32-bit (``trainer.mp``) the tokens are the plain implementation's greedy continuation, round after round."""
    d = write_model(TINY_B, 1, torch.float32)
    w = read_weights(d)
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, 1000, (n,), generator=g).tolist() for n in (9, 40, 1)]
    rounds, out = _sample_lm(["--hf_checkpoint", d, "--prompt_ids", json.dumps(prompts), "--temperature", "0", "--max_new_tokens", "16",
                              "--n_rounds", "2", "--trainer.mp", "p=f32,c=f32", "--engine.max_seqs", "4", "--engine.max_pages_per_seq", "8",
                              "--profile", "true"])
    assert sorted(rounds) == [0, 1] and "float32" in out
    assert out.count(" profile: ") == 2 and "waiting for the GPU" in out  # one line a round on where its time went
    for r in rounds.values():
        assert sorted(r) == [0, 1, 2]
        for i, p in enumerate(prompts):
            toks, reason = r[i]
            assert reason == "length" and toks == P.plain_greedy_generate(w, TINY_B, p, 16)


def test_command_line_from_a_yaml_file_with_overrides_in_bfloat16(tmp_path):
    """A configuration file plus dotted overrides (the reference's ``levanter.config.main`` surface,
    src/levanter/config.py:79-169): bfloat16 from ``trainer.mp``, engine options from the file and the command line, a
    stop sequence of token ids. Greedy tokens equal the plain implementation's (rounded to bfloat16 at the same places)
    wherever its two best logits are clearly apart."""
    d = write_model(TINY_A, 0, torch.bfloat16)
    w = read_weights(d)
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (5, 17, 33)]
    (tmp_path / "sample.yaml").write_text(
        "hf_checkpoint: %s\ntrainer:\n  mp: p=bfloat16,c=bfloat16\nengine:\n  max_seqs: 2\n  page_size: 32\n  max_pages_per_seq: 4\n"
        "  max_prefill_size: 11\nprompt_ids: %s\ntemperature: 0.0\nmax_new_tokens: 24\nn_rounds: 1\n" % (d, json.dumps(prompts)))
    rounds, out = _sample_lm(["--config_path", str(tmp_path / "sample.yaml"), "--engine.max_seqs", "3", "--max_new_tokens", "20"])
    assert "bfloat16" in out and sorted(rounds) == [0]
    clear = 0
    for i, p in enumerate(prompts):
        toks, reason = rounds[0][i]
        assert reason == "length" and len(toks) == 20  # the command line's value, not the file's
        clear += _check_greedy(w, TINY_A, p, toks, P.bf16_rounding, margin=2e-2)
    assert clear >= 45, clear  # of 60
    # a stop sequence: the 4th and 5th generated token of sequence 0 end it where they first appear one after the other
    first = rounds[0][0][0]
    stop = first[3:5]
    n_stop = next(n for n in range(1, 6) if P.plain_is_stop(prompts[0] + first[:n], [stop]))
    rounds2, _ = _sample_lm(["--config_path", str(tmp_path / "sample.yaml"), "--stop_ids", json.dumps(stop)])
    toks, reason = rounds2[0][0]
    assert reason == "stop" and toks == first[:n_stop]


def test_command_line_sampling_equals_the_python_entry_point():
    """With a temperature the command line draws what ``InferenceEngine.generate`` draws for the same keys: the key of
    request i is ``fold_in(make_key(engine.seed), i)``, as the command line derives it."""
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import InferenceEngine, Request, SeqDecodingParams
    from levanter_amd.sampling import fold_in, make_key

    d = write_model(TINY_A, 0, torch.float32)
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (3, 20)]
    rounds, _ = _sample_lm(["--hf_checkpoint", d, "--prompt_ids", json.dumps(prompts), "--temperature", "0.9", "--max_new_tokens", "12",
                            "--n_rounds", "1", "--trainer.mp", "p=f32,c=f32", "--engine.seed", "11", "--n_generations", "2",
                            "--engine.max_pages_per_seq", "8"])
    engine = InferenceEngine.from_pretrained(d, InferenceEngineConfig(compute_dtype="float32", seed=11, max_pages_per_seq=8))
    res = engine.generate([Request(prompt_tokens=p, request_id=i, n_generations=2,
                                   decode_params=SeqDecodingParams(max_num_tokens=len(p) + 12, temperature=0.9, key=fold_in(make_key(11), i)))
                           for i, p in enumerate(prompts)])
    assert [rounds[0][i][0] for i in range(4)] == res.tokens
    assert len({tuple(t) for t in res.tokens}) == 4  # generations of one request differ: it is sampling


def test_command_line_with_text_prompts_and_a_tokenizer_file():
    """Prompts and the stop sequence as text, as the reference's command takes them (src/levanter/main/sample_lm.py:97-121:
    the tokenizer encodes each prompt and the stop sequence without special tokens): a word-level ``tokenizer.json`` in the
    model folder. The ids are the tokenizer's, the tokens the plain implementation's greedy continuation up to the stop word,
    and the text lines are the tokenizer's decoding of them."""
    from tokenizers import Tokenizer, models, pre_tokenizers

    d = write_model(TINY_A, 0, torch.float32)
    w = read_weights(d)
    vocab = {f"w{i}": i for i in range(TINY_A["vocab_size"])}
    tok = Tokenizer(models.WordLevel(vocab=vocab, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(os.path.join(d, "tokenizer.json"))
    texts = ["w5 w17 w3 w400", "w77"]
    ids = [[5, 17, 3, 400], [77]]
    whole = [P.plain_greedy_generate(w, TINY_A, p, 12) for p in ids]
    stop_word = f"w{whole[0][4]}"  # the fifth generated token of prompt 0 ends it (or an earlier occurrence of the same word)
    expect = []
    for p, g in zip(ids, whole):
        n = next((n for n in range(1, len(g) + 1) if P.plain_is_stop(p + g[:n], [[whole[0][4]]])), len(g))
        expect.append(g[:n])
    rounds, out = _sample_lm(["--hf_checkpoint", d, "--prompts", json.dumps(texts), "--stop_sequence", stop_word, "--temperature", "0",
                              "--max_new_tokens", "12", "--n_rounds", "1", "--trainer.mp", "p=f32,c=f32", "--engine.max_pages_per_seq", "8"])
    for i, p in enumerate(ids):
        assert f"prompt {i} ({len(p)} tokens): {p}" in out
        toks, reason = rounds[0][i]
        assert toks == expect[i] and reason == ("stop" if P.plain_is_stop(p + toks, [[whole[0][4]]]) else "length")
        assert f"round 0 sequence {i} text: {' '.join(f'w{t}' for t in toks)}" in out
    assert rounds[0][0][1] == "stop" and len(rounds[0][0][0]) <= 5
