"""Norms. LayerNorm: (x - mean) / sqrt(var + eps) * weight + bias with the biased variance
(the reference builds it with ``hnn.LayerNorm.init(Embed, eps=layer_norm_epsilon, use_bias)``,
src/levanter/models/gpt2.py:228,230,263). Statistics are computed in 32-bit."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, Norm, StepContext
from .registry import NORMS
from .spec import PartSpec


@NORMS.register("layernorm")
class LayerNorm(Norm):
    graph_safe = True
    folds_pending = True

    rms = False

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.dim = int(spec.params["dim"])
        self.eps = float(spec.params["eps"])
        self.weight = tensors["weight"].to(env.device, torch.float32).contiguous()
        self.bias = tensors["bias"].to(env.device, torch.float32).contiguous() if spec.params.get("bias", True) else None

    def __call__(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        out = ctx.empty(n, self.dim)
        pending = ctx.take_pending(x)
        if pending is None:
            ctx.kernels.norm(x, self.weight, self.bias, self.eps, out, rows=rows, rms=self.rms)
        else:
            ctx.kernels.norm(x, self.weight, self.bias, self.eps, out, rows=rows, rms=self.rms, pending=pending)
        return out


@NORMS.register("rmsnorm")
class RmsNorm(LayerNorm):
    """x / sqrt(mean(x^2) + eps) * weight (+ bias): the same kernel without the mean."""

    rms = True
