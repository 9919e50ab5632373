"""Traces for replay tests: the same requests cut into steps in four ways, and the bookkeeping to
compare what a replay returns with the plain implementation's logits of whole sequences."""
from __future__ import annotations

import json
import random
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

PORTION_SIZES = [7, 2, 13, 3, 5, 2, 11, 4, 17, 2, 6]


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def want_all(n):
    return list(range(n))


def want_ends(n):
    """The first, the middle and the last two places of a portion: for models whose vocabulary makes every row costly."""
    return sorted({0, n // 2, max(0, n - 2), n - 1})


def _entry(rid, toks, start, n, want=want_all):
    return {"id": rid, "tokens": toks[start:start + n], "want": want(n)}


def trace_whole(reqs, prefix="w", want=want_all):
    """Each request alone, all its tokens in one step."""
    return [{"entries": [_entry(prefix + rid, toks, 0, len(toks), want)], "end": [prefix + rid]} for rid, toks in reqs.items()]


def trace_prefill_then_singles(reqs, n_single=32, prefix="s", want=want_all):
    """All but the last ``n_single`` tokens in one step, then one token a step."""
    steps = []
    for rid, toks in reqs.items():
        n = len(toks)
        k = max(1, n - n_single)
        steps.append({"entries": [_entry(prefix + rid, toks, 0, k, want)], "end": []})
        for i in range(k, n):
            steps.append({"entries": [_entry(prefix + rid, toks, i, 1)], "end": [prefix + rid] if i == n - 1 else []})
        if k == n:
            steps[-1]["end"] = [prefix + rid]
    return steps


def trace_portions(reqs, prefix="p", sizes=PORTION_SIZES, want=want_all):
    """Portions of changing size, down to two tokens."""
    steps = []
    j = 0
    for rid, toks in reqs.items():
        i, n = 0, len(toks)
        while i < n:
            size = min(sizes[j % len(sizes)], n - i)
            j += 1
            steps.append({"entries": [_entry(prefix + rid, toks, i, size, want)], "end": [prefix + rid] if i + size == n else []})
            i += size
    return steps


def trace_mixed(reqs, seed=0, max_live=4, prefix="m", decode_tail=12, sizes=(2, 3, 5, 7, 16, 17, 30), want=want_all):
    """Up to ``max_live`` live requests; portions of some beside single tokens of others in one step;
    requests are sometimes left out of a step; a finished request's place is taken by the next."""
    rng = random.Random(seed)
    waiting = [(prefix + rid, toks) for rid, toks in reqs.items()]
    live: Dict[str, Tuple[List[int], int]] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = (toks, 0)
        entries, end = [], []
        for rid in list(live):
            toks, i = live[rid]
            if len(live) > 1 and rng.random() < 0.25:
                continue  # left out of this step
            n = len(toks)
            if i >= n - decode_tail:
                size = 1
            else:
                size = min(rng.choice(list(sizes)), n - decode_tail - i)
            entries.append(_entry(rid, toks, i, size, want))
            if i + size == n:
                end.append(rid)
                del live[rid]
            else:
                live[rid] = (toks, i + size)
        if entries:
            rng.shuffle(entries)
            steps.append({"entries": entries, "end": end})
    return steps


def number(steps, start=0):
    for i, s in enumerate(steps):
        s["step"] = start + i
    return steps


def peak_tokens(steps, round_to=64) -> int:
    """The most tokens live requests hold at any time, each count rounded up to a multiple of ``round_to``."""
    held: Dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum((n + round_to - 1) // round_to * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def expected_rows(steps, plain_logits_of):
    """For every step with wanted places: the plain implementation's logits rows in the replay's order.
    ``plain_logits_of(request id)`` gives the [len, vocab] logits of the whole request."""
    done: Dict[str, int] = {}
    out = {}
    for s in steps:
        rows = []
        for e in s["entries"]:
            start = done.get(e["id"], 0)
            full = plain_logits_of(e["id"])
            rows += [full[start + w] for w in e["want"]]
            done[e["id"]] = start + len(e["tokens"])
        if rows:
            out[s["step"]] = torch.stack(rows)
    return out


def to_jsonl(steps) -> str:
    return "".join(json.dumps(s) + "\n" for s in steps)


# ---- the schedules of the reference's own paged-attention tests (tests/inference/test_paged_attention.py:293-442) ----
REFERENCE_RAGGED_SCHEDULE = [[4, 2], [0, 1], [0, 1], [2, 1], [1, 2], [1, 1]]  # tokens of request 0 and 1 in each step
REFERENCE_SLOT_ORDERS = [[0, 1], [1, 0], [2, 0], [0, 2], [2, 1]]              # the slots the two requests occupy
REFERENCE_PREFIX_SIZES = [1, 2, 3]
REFERENCE_CHUNK_SIZES = [1, 2, 3, 8]


def trace_two_requests(tokens0, tokens1, schedule, ids=("a", "b")):
    """Steps that bring ``schedule[i] = [n0, n1]`` tokens of two requests (0: the request is left out of the step)."""
    steps, off = [], [0, 0]
    toks = (tokens0, tokens1)
    for sizes in schedule:
        entries = []
        for r in (0, 1):
            if sizes[r]:
                entries.append(_entry(ids[r], toks[r], off[r], sizes[r]))
                off[r] += sizes[r]
        steps.append({"entries": entries, "end": [ids[r] for r in (0, 1) if sizes[r] and off[r] == len(toks[r])]})
    assert off == [len(tokens0), len(tokens1)]
    return number(steps)


def reference_chunk_schedule(prefix, chunk):
    """A prefix of both requests in one step, then four chunks each, as the reference's chunked-prefill test does."""
    return [[prefix, prefix]] + [[chunk, chunk]] * 4
