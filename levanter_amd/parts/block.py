"""Blocks: how the parts of a layer are arranged around the residual stream.
Pre-norm (src/levanter/models/gpt2.py:237-248): x += mixer(norm1(x)); x += feed_forward(norm2(x))."""
from __future__ import annotations

from typing import Dict

import torch

from .base import Block, CacheUnitView, Part, StepContext
from .registry import BLOCKS


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    roles = ("norm1", "mixer", "norm2", "feed_forward")
    defers_residual = True

    def __init__(self, parts: Dict[str, Part]):
        super().__init__(parts)
        self.norm1, self.mixer, self.norm2, self.feed_forward = (parts[r] for r in self.roles)

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        # a product that the part before has left unfinished is folded into the norm that follows it, or finished first
        if not self.norm1.folds_pending:
            ctx.settle()
        self.mixer.forward(self.norm1(x, ctx), x, ctx, unit, writes_cache)
        if not self.norm2.folds_pending:
            ctx.settle()
        self.feed_forward.forward(self.norm2(x, ctx), x, ctx)
