"""Blocks: how two norms, a mixer and a feed-forward are arranged around the residual stream.
Pre-norm (src/levanter/models/gpt2.py:237-248): x += mixer(norm1(x)); x += feed_forward(norm2(x))."""
from __future__ import annotations

import torch

from .base import Block, CacheUnitView, FeedForward, Mixer, Norm, StepContext
from .registry import BLOCKS


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward):
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.norm1, self.mixer, self.norm2, self.feed_forward))

    def forward(self, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        self.mixer.forward(self.norm1(x, ctx), x, ctx, unit, writes_cache)
        self.feed_forward.forward(self.norm2(x, ctx), x, ctx)
