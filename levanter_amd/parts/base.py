"""Interfaces of the parts and what a part sees of a step.

Every part is built from ``(spec, tensors, env)``: its ``PartSpec`` (sizes and constants), a
dict from its local parameter names to loaded tensors, and the ``BuildEnv`` (compute dtype,
device, kernel library). No part knows which model it is in.

The residual stream ``x`` is float32 ``[T, dim]`` in every precision; a norm turns it into the
compute dtype ``h``; mixers and feed-forwards add their result to ``x`` in place.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional

import torch

from levanter_amd.parts.spec import PartSpec


@dataclass
class BuildEnv:
    dtype: torch.dtype
    device: torch.device
    kernels: Any


@dataclass
class AttentionMeta:
    """Device-side description of the step's tokens for the attention kernels."""

    positions: torch.Tensor  # int32 [T] absolute position of each token
    token_seq: torch.Tensor  # int32 [T] row of the step's block tables (= index of the request in the step)
    prefill_tiles: Optional[torch.Tensor]  # int32 [n, 2]: first token and row count of each tile of a run longer than one token
    n_prefill_tiles: int
    decode_tokens: Optional[torch.Tensor]  # int32 [n]: tokens that are a run of their own
    n_decode: int
    max_kv_len: int  # the longest key range any token of the step reads
    _workspaces: Dict[Any, torch.Tensor] = field(default_factory=dict)
    plans: Dict[Any, Any] = field(default_factory=dict)
    """The kernel library's notes on this step (what it has checked and decided once for all layers of a cache group)."""

    def workspace(self, nbytes: int, device) -> Optional[torch.Tensor]:
        if nbytes <= 0:
            return None
        ws = self._workspaces.get("ws")
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._workspaces["ws"] = ws
        return ws


@dataclass
class GroupView:
    """One cache group in this step."""

    page_size: int
    block_tables: torch.Tensor  # int32 [S, blocks]: page ids of the step's requests, -1 where none
    dest: torch.Tensor  # int32 [T]: page * page_size + offset where each new token's keys and values go


@dataclass
class CacheUnitView:
    """What a mixer gets of its cache unit in this step: pages (paged units) or state (slot units)."""

    k_pages: Optional[torch.Tensor] = None
    v_pages: Optional[torch.Tensor] = None
    group: Optional[GroupView] = None
    state: Optional[torch.Tensor] = None  # [slots, *shape]; rows ctx.seq_slots belong to the step's requests


@dataclass
class StepContext:
    """What the parts see of one step. ``host`` holds the same facts as Python lists for parts that
    steer from the host (run lengths, first positions, slots)."""

    kernels: Any
    dtype: torch.dtype
    device: torch.device
    n_tokens: int
    tokens: torch.Tensor  # int32 [T]
    attention: AttentionMeta
    seq_slots: torch.Tensor  # int32 [S] state slot of each request in the step
    host: Dict[str, Any]  # "run_lengths", "first_positions", "slots": lists, one entry per request in the step
    token_slots: Optional[torch.Tensor] = None
    """int32 [T]: the state slot of each token's request, -1 for the padding tokens of a replayed step (they belong to
    nobody: a mixer with state of its own must not count them). With ``attention.positions`` and
    ``attention.token_seq`` this is all a state mixer needs on the device, so that it can be ``graph_safe``."""
    units: Dict[int, CacheUnitView] = field(default_factory=dict)
    pending: Any = None
    """A product into the residual stream that its kernel has not finished (``kernels.PendingSum``): the next norm of
    that tensor folds the rest in, anything else calls ``settle()`` first. Only set while ``may_defer`` is True."""
    may_defer: bool = False
    """Set by the decoder around blocks that say ``defers_residual``: the parts of such a block promise that after a
    product marked ``final`` they do not touch the residual stream again in their ``forward``."""

    def empty(self, rows: int, cols: int, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return torch.empty((rows, cols), dtype=dtype or self.dtype, device=self.device)

    def settle(self) -> None:
        """Finish what ``pending`` describes, if anything: afterwards the residual stream is up to date."""
        if self.pending is not None:
            pending, self.pending = self.pending, None
            self.kernels.finish(pending)

    def take_pending(self, x: torch.Tensor):
        """The unfinished product into ``x`` for a norm that folds it in (None if there is none; one into another
        tensor is settled)."""
        pending = self.pending
        if pending is None:
            return None
        self.pending = None
        if pending.out is x:
            return pending
        self.kernels.finish(pending)
        return None


class Part:
    kind: str = ""

    graph_safe = False
    """True if the part only launches work whose shape is fixed by the step's sizes and reads everything that
    changes from step to step (tokens, positions, tables) from device memory: such work can be recorded once into
    a HIP graph and replayed. A part that steers from the host (``ctx.host``, data-dependent shapes, copies to the
    CPU) leaves it False, and a model with such a part runs every step eagerly. Blocks answer for their members."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        self.spec = spec
        self.env = env


class Norm(Part):
    """``__call__(x_f32 [T, dim], ctx, rows=None) -> h [T or len(rows), dim]`` in the compute dtype.
    ``folds_pending``: the norm looks at ``ctx.take_pending(x)`` itself and hands it to its kernel; for one that does
    not (the default) the block or the decoder calls ``ctx.settle()`` before it runs."""

    folds_pending = False

    def __call__(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Two hooks; a position encoding uses one of them.

    ``embedding_table()``: a table ``[positions, dim]`` whose row is added to the token embedding, or None.
    ``rotate(q, k, ctx)``: change queries and keys in place before the cache write (identity by default).
    ``max_positions``: the largest sequence length it allows, or None."""

    max_positions: Optional[int] = None

    def embedding_table(self) -> Optional[torch.Tensor]:
        return None

    def rotate(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        return None


class Mixer(Part):
    """Mixes information between the tokens of a request.

    ``cache_requirement()``: ``PagedKv``, ``SlotState`` or None: what one cache unit of it holds.
    ``forward(h, x, ctx, unit, writes_cache)``: adds the mixer's output for ``h`` (compute dtype
    ``[T, dim]``) to the residual ``x`` (float32 ``[T, dim]``) in place; reads (and, if
    ``writes_cache``, first writes) ``unit``."""

    def cache_requirement(self):
        return None

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        raise NotImplementedError


class FeedForward(Part):
    """``forward(h, x, ctx)``: adds the feed-forward's output for ``h`` to the residual ``x`` in place."""

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        raise NotImplementedError


class Block:
    """Arranges the parts of a layer around the residual stream. Built from ``parts``: role -> built part, with the
    roles its description names; ``roles`` lists the ones this block cannot do without. One plan entry has one
    cache unit: ``cache_requirement()`` says what it holds (by default what the part in the role ``mixer`` asks for).
    ``forward(x, ctx, unit, writes_cache)`` updates ``x`` in place."""

    kind: str = ""
    roles: tuple = ()
    defers_residual = False
    """True: this block only reads the residual stream through norms (after ``ctx.settle()`` unless they fold pending
    sums in themselves) and through its parts, so a part's last product may leave its sum to the next norm."""

    def __init__(self, parts: Dict[str, Part]):
        missing = [r for r in self.roles if r not in parts]
        if missing:
            raise ValueError(f"block {self.kind!r} needs the parts {', '.join(self.roles)}; the description lacks {', '.join(missing)}")
        self.parts = dict(parts)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts.values())

    def cache_requirement(self):
        mixer = self.parts.get("mixer")
        return None if mixer is None else mixer.cache_requirement()

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        raise NotImplementedError


class Embedding(Part):
    """``__call__(ctx) -> x`` float32 ``[T, dim]``: the residual stream's first value, from ``ctx.tokens`` (and
    positions, if the embedding has a position encoding). ``table``: the token table ``[vocab, dim]`` in the compute
    dtype, for a head that is tied to it (None if there is no such table). ``max_positions``: the largest sequence
    length it allows, or None."""

    table: Optional[torch.Tensor] = None
    max_positions: Optional[int] = None

    def __call__(self, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """``__call__(h [R, dim], ctx) -> logits float32 [R, vocab]``. ``bind(embedding)`` is called once when the
    model is built: a tied head takes the embedding's table there; others ignore it."""

    def bind(self, embedding: Embedding) -> None:
        return None

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError
