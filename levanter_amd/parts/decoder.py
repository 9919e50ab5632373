"""DecoderLm: a runnable model built from a ``ModelSpec``.

Embedding (token table + position encoding), layers of parts, the plan (the order in which
layers run and which cache unit each reads), the final norm and the head. The reference wires
the same sequence for paged decoding in src/levanter/models/llama.py:346-363,404-432,589-633
(per-layer cache, logits from the packed positions); the GPT-2 mathematics is
src/levanter/models/gpt2.py:237-248,268-273,345-362.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .base import BuildEnv, StepContext
from .embedding import nested_tensors
from .registry import BLOCKS, part_class
from .spec import ModelSpec, PartSpec


class DecoderLm:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        self.spec = spec
        self.env = env
        self.vocab_size = spec.vocab_size
        self.dim = spec.dim

        def build(part: PartSpec, family: str = ""):
            return part_class(part.kind, part.family or family)(part, nested_tensors(part, tensors), env)

        self.embedding = build(spec.embedding, "embedding")
        self.blocks = [BLOCKS.get(layer.block)({role: build(part) for role, part in layer.parts.items()}) for layer in spec.layers]
        self.plan = list(spec.plan)
        self.final_norm = build(spec.final_norm, "norm")
        self.head = build(spec.head, "head")
        self.head.bind(self.embedding)
        self._check_plan()

    def _check_plan(self) -> None:
        owners: Dict[int, int] = {}
        for i, e in enumerate(self.plan):
            if not 0 <= e.layer < len(self.blocks):
                raise ValueError(f"plan entry {i} names layer {e.layer}, the model has {len(self.blocks)}")
            if e.writes_cache:
                if e.cache in owners:
                    raise ValueError(f"plan entries {owners[e.cache]} and {i} both write cache unit {e.cache}")
                owners[e.cache] = i
        for i, e in enumerate(self.plan):
            if not e.writes_cache:
                if e.cache not in owners or owners[e.cache] > i:
                    raise ValueError(f"plan entry {i} reads cache unit {e.cache} before any entry has written it")
                a = self.blocks[self.plan[owners[e.cache]].layer].cache_requirement()
                b = self.blocks[e.layer].cache_requirement()
                if a != b:
                    raise ValueError(f"plan entry {i} reads cache unit {e.cache}, whose owner keeps something else ({a} vs {b})")

    @property
    def graph_safe(self) -> bool:
        """Every part agrees to be replayed from a HIP graph (a block answers for its members)."""
        return all(getattr(p, "graph_safe", False) for p in (self.embedding, *self.blocks, self.final_norm, self.head))

    @property
    def max_positions(self) -> Optional[int]:
        m = self.spec.max_positions
        e = self.embedding.max_positions
        if m is None:
            return e
        return m if e is None else min(m, e)

    def cache_requirements(self) -> List[Tuple[int, object]]:
        """(cache unit, requirement) of every unit that a plan entry writes."""
        return [(e.cache, self.blocks[e.layer].cache_requirement()) for e in self.plan if e.writes_cache]

    def forward(self, ctx: StepContext, logit_rows: torch.Tensor) -> torch.Tensor:
        """Run the step's tokens through the plan; float32 logits ``[len(logit_rows), vocab]``."""
        hold = getattr(ctx.kernels, "hold_stream", None)
        if hold is not None:
            hold()  # hundreds of launches on the one current stream
        try:
            return self._forward(ctx, logit_rows)
        finally:
            if hold is not None:
                ctx.kernels.release_stream()

    def _forward(self, ctx: StepContext, logit_rows: torch.Tensor) -> torch.Tensor:
        x = self.embedding(ctx)
        for e in self.plan:
            block = self.blocks[e.layer]
            ctx.may_defer = bool(block.defers_residual)
            if not ctx.may_defer:
                ctx.settle()  # this block may read the residual stream in ways of its own
            block.forward(x, ctx, ctx.units[e.cache], e.writes_cache)
        ctx.may_defer = False
        if logit_rows.numel() == 0:
            ctx.pending = None  # nobody reads the residual stream any more
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=ctx.device)
        if not self.final_norm.folds_pending:
            ctx.settle()
        h = self.final_norm(x, ctx, rows=logit_rows)
        return self.head(h, ctx)

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for obj in self._walk(self):
            if isinstance(obj, torch.Tensor) and obj.data_ptr() not in seen:
                seen.add(obj.data_ptr())
                total += obj.numel() * obj.element_size()
        return total

    def _walk(self, obj, depth=0):
        if isinstance(obj, torch.Tensor):
            yield obj
        elif isinstance(obj, (list, tuple)):
            for o in obj:
                yield from self._walk(o, depth + 1)
        elif hasattr(obj, "__dict__") and depth < 6 and not isinstance(obj, (ModelSpec, PartSpec, BuildEnv)):
            for k, v in vars(obj).items():
                if k in ("spec", "env"):
                    continue
                yield from self._walk(v, depth + 1)
