"""Heads: from the final norm's rows to float32 logits. Tied: logits = h . table^T with the token
table (src/levanter/models/gpt2.py:361-362, src/levanter/models/lm_model.py:210)."""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildEnv, Head, StepContext
from .linear import Linear
from .registry import HEADS
from .spec import PartSpec


@HEADS.register("tied_head")
class TiedHead(Head):
    graph_safe = True

    """Uses the embedding's table (taken in ``bind``); holds no second copy."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.table = None

    def bind(self, embedding) -> None:
        if embedding.table is None:
            raise ValueError("a tied head needs an embedding with a token table")
        self.table = embedding.table  # [vocab, dim], compute dtype

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        logits = ctx.empty(h.shape[0], self.table.shape[0], torch.float32)
        ctx.kernels.linear(h, self.table, None, logits)
        return logits


@HEADS.register("linear_head")
class LinearHead(Head):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.proj = Linear(tensors["weight"], tensors.get("bias"), spec.params.get("weight_layout", "out_in"), env)

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return self.proj(h, ctx, out_dtype=torch.float32)
