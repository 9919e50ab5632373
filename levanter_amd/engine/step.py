"""The step function: one batch of (request, its next tokens) through the model, from the cache.

The reference's counterpart is ``model.decode(tokens, cache, batch_info, pos_ids)``
(src/levanter/models/llama.py:589-633) fed by ``PageTable.allocate_for_seq`` and
``PageBatchInfo`` (src/levanter/inference/page_table.py:142-324,508-542): each request
contributes a contiguous run of tokens whose positions continue its cache, pages are taken
lazily for the positions the run reaches, every new token gets the destination
``page * page_size + position % page_size``, and attention sees ``kv_len - q_len`` earlier
tokens plus the run itself. Here the batch has exactly the tokens it is given (no padding), the
tables are built on the host and go to the GPU in one copy, and only the wanted rows pass the
final norm and the head.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from levanter_amd.cache import NO_PAGE, CacheManager, OutOfPages, SequenceHandle
from levanter_amd.kernels.staging import pinned_pool
from levanter_amd.parts.base import AttentionMeta, BuildEnv, CacheUnitView, GroupView, StepContext
from levanter_amd.parts.decoder import DecoderLm



@dataclass
class StepEntry:
    """A request's part in a step: its next tokens and the places among them whose logits are wanted."""

    handle: SequenceHandle
    tokens: Sequence[int]
    want: Sequence[int] = ()


class StepError(ValueError):
    """A step that cannot run: a bad token id, a position beyond the model's range, a bad ``want``."""


class ModelRunner:
    """Owns the model, the cache manager's device tensors and the step function."""

    def __init__(self, model: DecoderLm, cache: CacheManager, env: BuildEnv, allocate: bool = True, use_graphs: bool = True):
        self.model = model
        self.cache = cache
        self.env = env
        if allocate:
            cache.allocate_tensors(env.dtype, env.device)
        self._workspaces: Dict[object, torch.Tensor] = {}
        self._graphs: Dict[tuple, object] = {}
        # rows of one attention tile of a run longer than one token: the kernel library's choice
        self.prefill_tile_rows = int(getattr(env.kernels, "prefill_tile_rows", 64))
        self.use_graphs = bool(use_graphs) and env.device.type == "cuda" and getattr(model, "graph_safe", False)
        limit = cache.page_size * cache.max_pages_per_seq
        mp = model.max_positions
        self.max_len = limit if mp is None else min(limit, mp)

    # ------------------------------------------------------------------------------------
    def pages_needed(self, entries: Sequence[StepEntry]) -> List[int]:
        """Pages each group would have to find for these entries."""
        return [sum(g.blocks_needed(e.handle.slot, e.handle.length, e.handle.length + len(e.tokens)) for e in entries)
                for g in self.cache.groups]

    def fits(self, entries: Sequence[StepEntry]) -> bool:
        return all(n <= g.pool.n_free for n, g in zip(self.pages_needed(entries), self.cache.groups))

    def _validate(self, entries: Sequence[StepEntry]) -> None:
        seen = set()
        v = self.model.vocab_size
        for e in entries:
            n = len(e.tokens)
            rid = e.handle.request_id
            if e.handle.closed:
                raise StepError(f"request {rid!r} has ended")
            if e.handle.slot in seen:
                raise StepError(f"request {rid!r} appears twice in one step")
            seen.add(e.handle.slot)
            if n == 0:
                raise StepError(f"request {rid!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < v:
                    raise StepError(f"request {rid!r}: token id {t} is outside the vocabulary of {v}")
            if e.handle.length + n > self.max_len:
                raise StepError(f"request {rid!r} would reach {e.handle.length + n} tokens; the limit is {self.max_len} "
                                f"(positions of the model and page_size * max_pages_per_seq)")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {rid!r}: wanted place {w} is not among its {n} tokens")

    # ------------------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], copy_out: bool = True, token_feed=None) -> torch.Tensor:
        """Run the entries as one batch. Returns float32 logits [wanted, vocab] in the order of the
        entries and of their ``want``. Raises ``OutOfPages`` (nothing changed) if a pool is too small.
        ``copy_out=False`` may return a buffer that the next step overwrites (the sampler reads it at once).
        ``token_feed = (device_tokens int32 [R], rows, n)``: the first n entries are single tokens that are not known on
        the host yet; entry i's token is ``device_tokens[rows[i]]`` (``rows`` None: ``device_tokens[i]``), the sampler's
        output of the step before, put in place on the device after the step's tables have been uploaded."""
        entries = list(entries)
        self._validate(entries)
        if token_feed is not None and (token_feed[2] > len(entries) or any(len(e.tokens) != 1 for e in entries[:token_feed[2]])):
            raise StepError("tokens can be fed from the device to the step's first entries only, each of a single token")
        if not entries:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.env.device)
        if not self.fits(entries):
            need = self.pages_needed(entries)
            raise OutOfPages("out of free pages: the step needs " + ", ".join(
                f"{n} of group {g.index}'s {g.pool.n_free} free" for n, g in zip(need, self.cache.groups)))
        extended: List[StepEntry] = []
        try:
            for e in entries:
                self.cache.extend(e.handle, len(e.tokens))
                extended.append(e)
            graphable = self.use_graphs and all(len(e.tokens) == 1 for e in entries)
            mixed = self._mixed_step_shape(entries) if self.use_graphs and not graphable else None
            batch = self._build_host(entries, pad_blocks=GRAPH_BLOCK_BUCKET if graphable else 1, pad_batch=graphable, mixed=mixed)
            if graphable or mixed is not None:
                logits = self._run_graphed(batch, token_feed)[:batch.n_rows_real]
                if copy_out:
                    logits = logits.clone()
            else:
                dev = self._upload(batch.host)
                self._feed_tokens(dev, batch, token_feed)
                logits = self.model.forward(self._make_ctx(dev, batch, self._workspaces), batch.rows_view)
        except BaseException:  # the step did not happen: its pages go back
            for e in extended:
                self.cache.retract(e.handle, len(e.tokens))
            raise
        for e in entries:
            self.cache.advance(e.handle, len(e.tokens))
        return logits

    # ------------------------------------------------------------------------------------
    def _mixed_step_shape(self, entries: Sequence[StepEntry]) -> Optional["MixedShape"]:
        """The shape that a step of prompt portions beside single tokens is filled up to, so that serving meets a handful
        of such shapes and can replay them as graphs: the single tokens to a multiple of ``MIXED_DECODE_BUCKET`` (with
        ghosts, as in steps of single tokens), room for up to ``MIXED_MAX_PORTIONS`` portions (request rows, wanted rows
        and the partial attention tiles they may add: empty tiles fill the rest), block tables at their full width. The
        portions' token count stays exact: a scheduler fills its budget, so most steps of a busy engine have the same.
        None: this step has more portions or more wanted rows than the shape holds, or so many tokens that the host's
        launches are a small part of it (a recorded graph keeps its activations for as long as it lives), and runs as it is."""
        portions = [len(e.tokens) for e in entries if len(e.tokens) > 1]
        if not 1 <= len(portions) <= MIXED_MAX_PORTIONS:
            return None
        singles = len(entries) - len(portions)
        n_decode = -(-singles // MIXED_DECODE_BUCKET) * MIXED_DECODE_BUCKET
        # the GPU's time for a step grows with tokens x width^2, the host's with the number of launches alone
        if (sum(portions) + n_decode) * self.model.dim ** 2 > MIXED_GRAPH_MAX_WORK:
            return None
        shape = MixedShape(n_decode=n_decode, n_seqs=n_decode + MIXED_MAX_PORTIONS, n_rows=n_decode + MIXED_MAX_PORTIONS,
                           n_tiles=sum(portions) // self.prefill_tile_rows + MIXED_MAX_PORTIONS)
        if sum(len(e.want) for e in entries) > shape.n_rows:
            return None
        return shape

    def _build_host(self, entries: Sequence[StepEntry], pad_blocks: int = 1, pad_batch: bool = False,
                    mixed: Optional["MixedShape"] = None) -> "HostBatch":
        """Everything the GPU needs to know about the step, in one int32 buffer with a layout that
        depends only on (tokens, requests, wanted rows, tiles, single tokens, blocks per request).

        ``pad_batch`` (steps of single tokens that may be replayed as a graph): the batch is filled up to
        ``graph_batch_bucket`` tokens with ghosts, so that a serving run whose requests end one by one meets a
        handful of shapes instead of one per batch size. A ghost is a token 0 at position 0 that reads the first
        request's first key, is written nowhere (destination -1) and whose logits (of its own row) nobody reads."""
        cache, ps = self.cache, self.cache.page_size
        S = len(entries)
        T = sum(len(e.tokens) for e in entries)
        tokens = np.empty(T, np.int32)
        positions = np.empty(T, np.int32)
        token_seq = np.empty(T, np.int32)
        seq_slots = np.empty(S, np.int32)
        rows: List[int] = []
        tile_list: List[tuple] = []  # (last position it reads, first token, rows)
        decode: List[int] = []
        run_lengths, first_positions = [], []
        max_blocks = 1
        t0 = 0
        for s, e in enumerate(entries):
            n, start = len(e.tokens), e.handle.length
            tokens[t0:t0 + n] = np.asarray(e.tokens, dtype=np.int64)
            positions[t0:t0 + n] = np.arange(start, start + n)
            token_seq[t0:t0 + n] = s
            seq_slots[s] = e.handle.slot
            rows.extend(t0 + int(w) for w in e.want)
            if n == 1:
                decode.append(t0)
            else:
                for r0 in range(0, n, self.prefill_tile_rows):
                    nr = min(self.prefill_tile_rows, n - r0)
                    tile_list.append((start + r0 + nr, t0 + r0, nr))
            run_lengths.append(n)
            first_positions.append(start)
            max_blocks = max(max_blocks, (start + n + ps - 1) // ps)
            t0 += n
        n_real_tokens, n_rows_real = T, len(rows)
        if pad_batch and rows:
            ghosts = graph_batch_bucket(T) - T
            if ghosts > 0:
                tokens = np.concatenate([tokens, np.zeros(ghosts, np.int32)])
                positions = np.concatenate([positions, np.zeros(ghosts, np.int32)])
                token_seq = np.concatenate([token_seq, np.zeros(ghosts, np.int32)])
                seq_slots = np.concatenate([seq_slots, np.full(ghosts, seq_slots[0], np.int32)])
                decode.extend(range(T, T + ghosts))
                rows.extend(range(T, T + ghosts))  # a ghost's logits are its own row's: no row is wanted twice
                S += ghosts
                T += ghosts
        if mixed is not None:
            ghosts = mixed.n_decode - len(decode)
            if ghosts > 0:  # ghost tokens as above, each with a request row of its own (a copy of the first request's)
                tokens = np.concatenate([tokens, np.zeros(ghosts, np.int32)])
                positions = np.concatenate([positions, np.zeros(ghosts, np.int32)])
                token_seq = np.concatenate([token_seq, np.arange(S, S + ghosts, dtype=np.int32)])
                decode.extend(range(T, T + ghosts))
                S += ghosts
                T += ghosts
            seq_slots = np.concatenate([seq_slots, np.full(mixed.n_seqs - len(seq_slots), seq_slots[0], np.int32)])  # rows no token names
            S = mixed.n_seqs
            # wanted rows nobody reads: a ghost's own row where there is one (the norm before the head takes a row twice)
            rows.extend([n_real_tokens + i % ghosts if ghosts > 0 else 0 for i in range(mixed.n_rows - len(rows))])
            tile_list.extend([(0, 0, 0)] * (mixed.n_tiles - len(tile_list)))  # empty tiles: their workgroups return at once
            max_blocks = cache.max_pages_per_seq
        # the attention kernel pairs tile i with tile n - 1 - i: sorted by falling key range, pairs have equal work
        tile_list.sort(key=lambda x: -x[0])
        tiles: List[int] = [v for _, first, nr in tile_list for v in (first, nr)]
        if pad_blocks > 1:
            max_blocks = min((max_blocks + pad_blocks - 1) // pad_blocks * pad_blocks, cache.max_pages_per_seq)
        n_groups = len(cache.groups)
        token_slots = seq_slots[token_seq].astype(np.int32)
        token_slots[n_real_tokens:] = -1  # ghosts belong to nobody: a mixer with state of its own leaves them out
        sizes = [T, T, T, S, len(rows), len(tiles), len(decode), T] + [S * max_blocks, T] * n_groups
        offs = np.concatenate([[0], np.cumsum([(x + 3) // 4 * 4 for x in sizes])]).astype(np.int64)
        host = np.zeros(int(offs[-1]), np.int32)
        for i, arr in enumerate((tokens, positions, token_seq, seq_slots, rows, tiles, decode, token_slots)):
            host[offs[i]:offs[i] + sizes[i]] = arr
        for gi, g in enumerate(cache.groups):
            bt = g.block_tables[seq_slots, :max_blocks]
            host[offs[N_FIXED + 2 * gi]:offs[N_FIXED + 2 * gi] + S * max_blocks] = bt.reshape(-1)
            pages = g.block_tables[seq_slots[token_seq], positions // ps]
            assert (pages[:n_real_tokens] != NO_PAGE).all(), "a new token has no page"
            dest = pages * ps + positions % ps
            dest[n_real_tokens:] = -1  # ghosts are written nowhere
            host[offs[N_FIXED + 1 + 2 * gi]:offs[N_FIXED + 1 + 2 * gi] + T] = dest
        return HostBatch(host=host, sizes=sizes, offs=[int(o) for o in offs], n_tokens=T, n_seqs=S, n_rows=len(rows),
                         n_tiles=len(tiles) // 2, n_decode=len(decode), max_blocks=max_blocks, max_kv=max_blocks * ps,
                         run_lengths=run_lengths, first_positions=first_positions, slots=[int(x) for x in seq_slots[:len(entries)]],
                         n_rows_real=n_rows_real)

    def _make_ctx(self, dev: torch.Tensor, b: "HostBatch", workspaces: Dict[object, torch.Tensor]) -> StepContext:
        def view(i):
            return dev[b.offs[i]:b.offs[i] + b.sizes[i]]

        cache, ps = self.cache, self.cache.page_size
        meta = AttentionMeta(
            positions=view(1), token_seq=view(2),
            prefill_tiles=view(5).view(-1, 2) if b.n_tiles else None, n_prefill_tiles=b.n_tiles,
            decode_tokens=view(6) if b.n_decode else None, n_decode=b.n_decode,
            max_kv_len=b.max_kv, _workspaces=workspaces)
        ctx = StepContext(kernels=self.env.kernels, dtype=self.env.dtype, device=self.env.device, n_tokens=b.n_tokens,
                          tokens=view(0), attention=meta, seq_slots=view(3), token_slots=view(7),
                          host={"run_lengths": b.run_lengths, "first_positions": b.first_positions, "slots": b.slots})
        group_views = [GroupView(page_size=ps, block_tables=view(N_FIXED + 2 * gi).view(b.n_seqs, b.max_blocks),
                                 dest=view(N_FIXED + 1 + 2 * gi)) for gi in range(len(cache.groups))]
        for unit, g in cache.group_of_unit.items():
            i = g.unit_pos[unit]
            ctx.units[unit] = CacheUnitView(k_pages=None if g.k_pages is None else g.k_pages[i],
                                            v_pages=None if g.v_pages is None else g.v_pages[i], group=group_views[g.index])
        for unit, t in cache.state.tensors.items():
            ctx.units[unit] = CacheUnitView(state=t)
        for e in self.model.plan:  # units whose mixers keep nothing still need a view
            ctx.units.setdefault(e.cache, CacheUnitView())
        b.rows_view = view(4)
        return ctx

    def _upload(self, host: np.ndarray) -> torch.Tensor:
        if self.env.device.type == "cpu":
            return torch.from_numpy(host)
        return pinned_pool().upload(host, self.env.device)

    # ---- decode steps as HIP graphs --------------------------------------------------------
    def _feed_tokens(self, dev: torch.Tensor, b: "HostBatch", token_feed) -> None:
        """Entry i's token id (i < n) comes from ``device_tokens[rows[i]]``: these entries are the step's first tokens."""
        if token_feed is None:
            return
        device_tokens, rows, n = token_feed
        self.env.kernels.feed_tokens(dev[b.offs[0]:b.offs[0] + n], device_tokens, rows, n)

    def _run_graphed(self, b: "HostBatch", token_feed=None) -> torch.Tensor:
        """A step's kernel sequence depends only on its counts (tokens, requests, wanted rows, attention tiles, single
        tokens, blocks per request), which steps of single tokens and mixed steps are filled up to a few values of: the
        second time such a step comes it is captured into a HIP graph whose inputs live in a fixed device buffer; later
        steps copy their tables there and replay it."""
        key = (b.n_tokens, b.n_seqs, b.n_rows, b.n_tiles, b.n_decode, b.max_blocks)
        entry = self._graphs.get(key)
        if entry is None:  # first time: run eagerly (also loads every kernel the graph will need)
            self._graphs[key] = "seen"
            dev = self._upload(b.host)
            self._feed_tokens(dev, b, token_feed)
            return self.model.forward(self._make_ctx(dev, b, self._workspaces), b.rows_view)
        if entry == "seen":
            if len(self._graphs) > MAX_GRAPHS:
                self._graphs = {k: v for k, v in self._graphs.items() if v == "seen"}
            n = len(b.host)
            entry = _Graph(static=torch.zeros(n, dtype=torch.int32, device=self.env.device),
                           pinned=torch.zeros(n, dtype=torch.int32).pin_memory(), copied=torch.cuda.Event())
            entry.pinned.numpy()[:] = b.host
            entry.static.copy_(entry.pinned, non_blocking=True)
            self._feed_tokens(entry.static, b, token_feed)
            ctx = self._make_ctx(entry.static, b, {})
            torch.cuda.current_stream().synchronize()
            entry.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(entry.graph):
                entry.logits = self.model.forward(ctx, b.rows_view)
            self._graphs[key] = entry
        else:
            entry.copied.synchronize()  # the previous copy out of the pinned buffer is done
            entry.pinned.numpy()[:] = b.host
            entry.static.copy_(entry.pinned, non_blocking=True)
            self._feed_tokens(entry.static, b, token_feed)
        entry.copied.record()
        entry.graph.replay()
        return entry.logits


MIXED_DECODE_BUCKET = 16  # single tokens beside prompt portions are filled up to a multiple of this
MIXED_MAX_PORTIONS = 4    # prompt portions a replayable mixed step has room for
# Larger mixed steps are not recorded: the GPU's time dwarfs the host's, and a graph holds its activations. In tokens x width^2:
# 512 tokens of a 4,096-wide model (a GPT-2 XL step of any size, 227 tokens at 6,144 wide).
MIXED_GRAPH_MAX_WORK = 512 * 4096 ** 2

N_FIXED = 8  # arrays of the step's buffer ahead of the cache groups' (block tables, destinations)
GRAPH_BLOCK_BUCKET = 16  # block tables of graphed steps are padded to a multiple of this many pages
MAX_GRAPHS = 48


def graph_batch_bucket(n: int) -> int:
    """Batch size that a graphed step of ``n`` single tokens is filled up to: small batches stay as they are,
    larger ones go to the next multiple of 8 (the GEMM kernels work on row tiles of 16 anyway)."""
    return n if n <= 4 else (n + 7) // 8 * 8


@dataclass(frozen=True)
class MixedShape:
    """Counts that a step of prompt portions beside single tokens is filled up to (see ``_mixed_step_shape``)."""

    n_decode: int
    n_seqs: int
    n_rows: int
    n_tiles: int


@dataclass
class _Graph:
    static: torch.Tensor
    pinned: torch.Tensor
    copied: "torch.cuda.Event"
    graph: Optional["torch.cuda.CUDAGraph"] = None
    logits: Optional[torch.Tensor] = None


@dataclass
class HostBatch:
    host: np.ndarray
    sizes: List[int]
    offs: List[int]
    n_tokens: int
    n_seqs: int
    n_rows: int
    n_tiles: int
    n_decode: int
    max_blocks: int
    max_kv: int
    run_lengths: List[int]
    first_positions: List[int]
    slots: List[int]
    n_rows_real: int = 0
    rows_view: Optional[torch.Tensor] = None
