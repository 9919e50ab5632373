"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees; decides what happens when pages run out.

Reference: ``InferenceEngine`` (src/levanter/inference/engine.py:643-1258) admits FIFO with
head-of-line blocking when slots and pages for the prompt are free (:807-854), prefills whole
prompts in one step (:865-1017), then decodes every live sequence one token per round
(:539-633); a sequence ends when its length reaches ``max_num_tokens`` or its tokens end with a
stop sequence, and the ending token is emitted (src/levanter/inference/jit_scheduler.py:329-340,
engine.py:613); pages and slot are released at once (engine.py:242-256,778-800). When pages run
out during decoding the reference fails the whole call (src/levanter/inference/page_table.py:219-223).

Here: one step holds the running sequences' single tokens (at most ``max_tokens_per_round``)
beside portions of prompts (at most ``max_prefill_size`` prompt tokens from at most
``max_seqs_in_prefill`` requests, oldest first; a prompt is cut where the budget ends). When a
step cannot get its pages, prompt portions are shrunk first; if decoding alone does not fit, the
youngest running sequence is preempted: its pages are freed and it returns to the head of the
queue with all its tokens so far as its prompt (recompute). A sequence that cannot fit even
alone in the pool ends with an error of its own; the others go on.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, Deque, List, Optional, Sequence, Tuple

from levanter_amd.cache import CacheManager, SequenceHandle
from levanter_amd.config import InferenceEngineConfig

from .request import Request


def is_stop_signal(tokens: Sequence[int], stop_sequences: Optional[Sequence[Sequence[int]]]) -> bool:
    """Do the tokens end with one of the stop sequences? Empty sequences never match
    (src/levanter/inference/utils.py:46-64)."""
    if not stop_sequences:
        return False
    n = len(tokens)
    for seq in stop_sequences:
        k = len(seq)
        if 0 < k <= n and all(int(tokens[n - k + i]) == int(seq[i]) for i in range(k)):
            return True
    return False


@dataclass
class Sequence_:
    """One generation of one request: the scheduler's fixed-size record of it (the reference's
    ``DecodeState`` row, src/levanter/inference/jit_scheduler.py:66-117)."""

    request: Request
    child: int
    key: Tuple[int, int]
    order: int
    tokens: List[int]  # prompt, then generated
    prompt_len: int
    generated: List[int] = field(default_factory=list)
    logprobs: List[float] = field(default_factory=list)
    handle: Optional[SequenceHandle] = None
    done: bool = False
    finish_reason: str = ""
    n_preempted: int = 0
    last_step: int = 0
    """Number of the last planned step that held tokens of this sequence (who decodes next when a step cannot hold all)."""

    @property
    def n_cached(self) -> int:
        return 0 if self.handle is None else self.handle.length

    @property
    def n_pending(self) -> int:
        """Tokens known but not yet in the cache: the rest of the prompt, or the last sampled token."""
        return len(self.tokens) - self.n_cached


@dataclass
class PlannedEntry:
    seq: Sequence_
    tokens: List[int]
    wants_logits: bool


class Scheduler:
    def __init__(self, cache: CacheManager, cfg: InferenceEngineConfig, max_len: int):
        self.cache = cache
        self.cfg = cfg
        self.max_len = max_len
        self.waiting: Deque[Sequence_] = deque()
        self.running: List[Sequence_] = []
        self._arrivals = 0
        self._steps_since_admission = 0
        self._step_no = 0
        self.n_preemptions = 0

    # ---- intake -----------------------------------------------------------------------------
    def next_order(self) -> int:
        self._arrivals += 1
        return self._arrivals

    def add(self, seq: Sequence_) -> None:
        self.waiting.append(seq)

    @property
    def idle(self) -> bool:
        return not self.waiting and not self.running

    # ---- admission ----------------------------------------------------------------------------
    def _first_portion(self, seq: Sequence_) -> int:
        return min(seq.n_pending, self.cfg.imputed_max_prefill_size)

    def _pages_for(self, n_tokens: int) -> int:
        ps = self.cache.page_size
        return (n_tokens + ps - 1) // ps

    def _min_free_pages(self) -> int:
        return min((g.pool.n_free for g in self.cache.groups), default=1 << 30)

    def _admit(self) -> None:
        """FIFO with head-of-line blocking (engine.py:807-854): a request enters when a slot is free and
        the pools hold the pages of its first portion beside one page of growth per running sequence."""
        while self.waiting and self.cache.n_free_slots > 0:
            seq = self.waiting[0]
            need = self._pages_for(self._first_portion(seq)) + len(self.running)
            if self.running and need > self._min_free_pages():
                break
            self.waiting.popleft()
            seq.handle = self.cache.open((seq.request.request_id, seq.child))
            self.running.append(seq)

    # ---- one step ---------------------------------------------------------------------------------
    def plan(self) -> List[PlannedEntry]:
        """Decide the next step: admit, pick tokens under the budgets, make them fit the pools."""
        while True:
            if not self.running or self._steps_since_admission >= self.cfg.max_rounds or any(
                    s.n_cached < s.prompt_len for s in self.running):
                self._admit()
                self._steps_since_admission = 0
            entries, starved = self._pick()
            if not starved:
                if entries:
                    self._planned(entries)
                return entries
            # pages ran out: preempt the youngest running sequence, or fail the only one
            victim = max(self.running, key=lambda s: s.order)
            if len(self.running) == 1:
                pools = ", ".join(str(g.pool.n_pages) for g in self.cache.groups) or "none"
                self._finish(victim, f"error: out of pages (needs more than the pool holds: {pools} pages)")
                if not self.waiting:
                    return []
                continue
            self._preempt(victim)

    def _planned(self, entries: List[PlannedEntry]) -> None:
        self._steps_since_admission += 1
        self._step_no += 1
        for e in entries:
            e.seq.last_step = self._step_no

    @staticmethod
    def _turn(seq: Sequence_):
        """Who decodes first when ``max_tokens_per_round`` is below the number of decoding sequences: the one that
        has waited longest, then the oldest. The reference's queue of pending tokens rotates the same way
        (src/levanter/inference/jit_scheduler.py:524-577): what a round leaves over goes first in the next."""
        return (seq.last_step, seq.order)

    def _taker(self):
        """take(seq, n): count the pages that n more tokens of seq need against what the pools have left."""
        free = [g.pool.n_free for g in self.cache.groups]

        def take(seq: Sequence_, n: int) -> bool:
            need = [g.blocks_needed(seq.handle.slot, seq.handle.length, seq.handle.length + n) for g in self.cache.groups]
            if any(nd > fr for nd, fr in zip(need, free)):
                return False
            for i, nd in enumerate(need):
                free[i] -= nd
            return True

        return take, free

    def _pick_portions(self, entries: List[PlannedEntry], take, free) -> bool:
        """Prompt portions under the token budget, oldest request first, behind the entries already picked.
        Returns whether the step is starved (nothing picked at all because the pages ran out)."""
        budget = self.cfg.imputed_max_prefill_size
        n_prefill = 0
        for seq in sorted((s for s in self.running if s.n_cached < s.prompt_len), key=lambda s: s.order):
            if budget <= 0 or n_prefill >= self.cfg.max_seqs_in_prefill:
                break
            n = min(seq.n_pending, budget)
            while n > 0 and not take(seq, n):
                # shrink to what the free pages hold: up to the end of the last page that fits
                ps = self.cache.page_size
                room = min(free) * ps + (-seq.handle.length) % ps
                n = min(n - 1, room)
            if n <= 0:
                return not entries
            start = seq.n_cached
            entries.append(PlannedEntry(seq, seq.tokens[start:start + n], start + n == len(seq.tokens)))
            budget -= n
            n_prefill += 1
        return False

    def _pick(self) -> Tuple[List[PlannedEntry], bool]:
        take, free = self._taker()
        entries: List[PlannedEntry] = []
        starved = False
        decoding = [s for s in self.running if s.n_cached >= s.prompt_len and s.n_pending == 1]
        decoding.sort(key=self._turn)
        for seq in sorted(decoding[: self.cfg.imputed_max_tokens_per_round], key=lambda s: s.order):
            if take(seq, 1):
                entries.append(PlannedEntry(seq, [seq.tokens[-1]], True))
            else:
                starved = True
        starved = self._pick_portions(entries, take, free) or starved
        return entries, starved

    def plan_lookahead(self, pending: List[PlannedEntry]) -> Optional[Tuple[List[PlannedEntry], List[int]]]:
        """The step after ``pending`` (a launched step whose sampled tokens are not on the host yet), if it can be
        decided without them. Every request that ``pending`` samples a token for decodes that token next: its entry
        holds a placeholder, and its row among ``pending``'s sampled tokens is returned beside the entries (these
        entries come first). Prompt portions and admissions follow as in ``plan``, from what the host knows. Requests
        that end by length with ``pending``'s token are left out; one that ends by a stop sequence cannot be foreseen
        and is skipped when this step is committed (so are the pages and the slot it would have given back: the plan is
        made as if nobody ended). Sequences whose next token the host knows already (``max_tokens_per_round`` left them
        out of ``pending``) stand behind the fed ones; who decodes is decided by turns as in ``plan``. Nothing is
        preempted here. None: wait for the tokens and plan as usual."""
        if not pending or any(e.seq.done for e in pending):
            return None
        row_of: Dict[int, int] = {}
        for e in pending:
            if e.wants_logits:
                row_of[id(e.seq)] = len(row_of)
        fed = [s for s in self.running if id(s) in row_of
               and len(s.tokens) + 1 < min(s.request.decode_params.max_num_tokens, self.max_len)]  # else pending's token is its last
        known = [s for s in self.running if id(s) not in row_of and s.n_cached >= s.prompt_len and s.n_pending == 1]
        chosen = sorted(fed + known, key=self._turn)[: self.cfg.imputed_max_tokens_per_round]
        if self._steps_since_admission >= self.cfg.max_rounds or any(s.n_cached < s.prompt_len for s in self.running):
            self._admit()
            self._steps_since_admission = 0
        take, free = self._taker()
        entries: List[PlannedEntry] = []
        rows: List[int] = []
        for seq in sorted((s for s in chosen if id(s) in row_of), key=lambda s: s.order):
            if not take(seq, 1):
                return None  # pages run out: the ordinary plan decides whom to preempt
            entries.append(PlannedEntry(seq, [0], True))
            rows.append(row_of[id(seq)])
        for seq in sorted((s for s in chosen if id(s) not in row_of), key=lambda s: s.order):
            if not take(seq, 1):
                return None
            entries.append(PlannedEntry(seq, [seq.tokens[-1]], True))
        if self._pick_portions(entries, take, free) or not entries:
            return None
        self._planned(entries)
        return entries, rows

    def _preempt(self, seq: Sequence_) -> None:
        """Free the sequence's pages and slot; it re-enters at the head of the queue and recomputes
        the cache of all its tokens so far. Its generated tokens and sampling key are kept."""
        self.cache.close(seq.handle)
        seq.handle = None
        seq.prompt_len = len(seq.tokens)  # everything known is now prompt
        seq.n_preempted += 1
        self.n_preemptions += 1
        self.running.remove(seq)
        self.waiting.appendleft(seq)

    # ---- after the step ------------------------------------------------------------------------------
    def commit(self, entries: List[PlannedEntry], sampled: Sequence[int], logprobs: Sequence[float]) -> List[Sequence_]:
        """Append the sampled token of every entry that wanted one; finish and free. Returns the finished."""
        finished = []
        i = 0
        for e in entries:
            if not e.wants_logits:
                continue
            seq, tok, lp = e.seq, int(sampled[i]), float(logprobs[i])
            i += 1
            if seq.done:  # it ended by a stop sequence after this step had been launched ahead
                continue
            seq.tokens.append(tok)
            seq.generated.append(tok)
            seq.logprobs.append(lp)
            p = seq.request.decode_params
            if is_stop_signal(seq.tokens, p.stop_tokens):
                self._finish(seq, "stop")
            elif len(seq.tokens) >= min(p.max_num_tokens, self.max_len):
                self._finish(seq, "length")
            if seq.done:
                finished.append(seq)
        return finished

    def _finish(self, seq: Sequence_, reason: str) -> None:
        seq.done = True
        seq.finish_reason = reason
        if seq.handle is not None:
            self.cache.close(seq.handle)
            seq.handle = None
        if seq in self.running:
            self.running.remove(seq)

    def abort_all(self) -> None:
        for seq in list(self.running):
            self._finish(seq, "error: aborted")
        self.waiting.clear()
