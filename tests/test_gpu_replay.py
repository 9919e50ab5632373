"""Replay through bin/trace_run on the GPU, in 32-bit and in bfloat16: the same requests whole,
with the last 32 tokens one by one, in portions of changing size, and mixed with other requests in
a pool so small that pages are used again. All compared with the plain implementation."""
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

import plain_gpt2 as P
import traces as TR
from helpers import read_weights, write_model
from tiny_configs import TINY

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# 32-bit: differences of summation order only (the reference's own tolerance for paged attention on
# the CPU is 1e-4, tests/inference/test_paged_attention.py:140-142).
TOL_F32 = dict(rtol=1e-4, atol=1e-5)
# bfloat16 against the plain implementation that rounds to bfloat16 at the same places: what is left
# are accumulation order and roundings that fall on the other side (one bfloat16 step is 2^-8
# relative; activations of order 1 pass through a few dozen roundings).
TOL_BF16 = dict(rtol=2e-2, atol=8e-3)


def run_trace(model_dir, dtype, steps, max_tokens, extra=()):
    out = tempfile.mkdtemp(prefix="lev_trace_")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", out,
           "--max-tokens", str(max_tokens), *extra]
    p = subprocess.run(cmd, input=TR.to_jsonl(steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-3000:]
    assert p.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return out


def read_step(out, step, vocab):
    return torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, vocab))


LENGTHS = {"A": [70, 45, 100, 37, 64, 33], "B": [90, 130, 41, 200, 64, 17], "C": [130, 66, 35, 97, 64, 18]}


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_all_cuttings(name, dtype):
    raw, seed = TINY[name]
    check_all_cuttings(f"trace_run {name}", raw, seed, dtype, LENGTHS[name])


def check_all_cuttings(label, raw, seed, dtype, lengths, page_size=16):
    """The requests whole, with the last 32 tokens one by one, in portions of changing size and twice mixed in a pool
    of exactly the peak need, through ``bin/trace_run``; every wanted row against the plain implementation."""
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    d = write_model(raw, seed, store)
    weights = read_weights(d)
    reqs = TR.random_requests(raw["vocab_size"], lengths, seed + 10)
    rounding = P.bf16_rounding if dtype == "bfloat16" else (lambda x: x)
    plain = {rid: P.plain_logits(weights, raw, torch.tensor(t), rounding=rounding) for rid, t in reqs.items()}
    steps = TR.number(TR.trace_whole(reqs) + TR.trace_prefill_then_singles(reqs) + TR.trace_portions(reqs)
                      + TR.trace_mixed(reqs, seed=3) + TR.trace_mixed(reqs, seed=4, prefix="n"))
    max_tokens = TR.peak_tokens(steps, round_to=64 if 64 % page_size == 0 else page_size)  # whole pages of every request
    out = run_trace(d, dtype, steps, max_tokens, extra=() if page_size == 16 else ("--page-size", str(page_size)))
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    tol = TOL_F32 if dtype == "float32" else TOL_BF16
    worst = 0.0
    for s in steps:
        k = s["step"]
        assert (k in want) == os.path.exists(os.path.join(out, f"{k}.f32"))
        if k in want:
            got = read_step(out, k, raw["vocab_size"])
            worst = max(worst, float((got.double() - want[k]).abs().max()))
            torch.testing.assert_close(got.double(), want[k], **tol, msg=lambda m: f"step {k} {s['entries'][0]['id']}: {m}")
    print(f"{label} {dtype}: worst abs difference {worst:.3e}")
    if dtype == "bfloat16":
        # and against the 32-bit plain implementation: the greedy token agrees wherever its margin is clear
        plain32 = {rid: P.plain_logits(weights, raw, torch.tensor(t)) for rid, t in reqs.items()}
        want32 = TR.expected_rows(steps, lambda rid: plain32[rid[1:]])
        for k, w in want32.items():
            got = read_step(out, k, raw["vocab_size"])
            top2 = w.topk(2, dim=-1).values
            clear = (top2[:, 0] - top2[:, 1]) > 2e-2
            assert bool((got.argmax(-1)[clear] == w.argmax(-1)[clear]).all())
            assert float((torch.softmax(got.double(), -1) - torch.softmax(w, -1)).abs().max()) < 1e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_from_a_configuration_and_a_seed(dtype):
    """``--random-config`` with ``--seed`` in place of ``--model``: the weights are those a folder written from the same
    configuration and seed holds, so the logits are the same bits."""
    import json

    raw, seed = TINY["A"]
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    d = write_model(raw, seed, store)
    reqs = TR.random_requests(raw["vocab_size"], [40, 21], 3)
    steps = TR.number(TR.trace_portions(reqs))
    out_folder = run_trace(d, dtype, steps, 128)
    out = tempfile.mkdtemp(prefix="lev_trace_")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-config", json.dumps(raw), "--seed", str(seed), "--dtype", dtype,
           "--out", out, "--max-tokens", "128"]
    p = subprocess.run(cmd, input=TR.to_jsonl(steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-3000:]
    n = 0
    for s_ in steps:
        f = os.path.join(out_folder, f"{s_['step']}.f32")
        if os.path.exists(f):
            assert torch.equal(read_step(out, s_["step"], raw["vocab_size"]), read_step(out_folder, s_["step"], raw["vocab_size"]))
            n += 1
    assert n > 0
    p = subprocess.run(cmd[:2] + ["--dtype", dtype, "--out", out, "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "either --model or --random-config" in p.stderr
