"""A linear map as the parts hold it: the matrix ``[out, in]`` in the compute dtype, the bias in float32."""
from __future__ import annotations

from typing import Optional

import torch

from .base import BuildEnv, StepContext


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor], layout: str, env: BuildEnv):
        """``layout``: "in_out" (stored [in, out], as GPT-2 checkpoints do) or "out_in"."""
        if layout not in ("in_out", "out_in"):
            raise ValueError(f"unknown weight layout {layout!r}")
        w = weight.to(env.device)
        if layout == "in_out":
            w = w.t()
        self.weight = w.to(env.dtype).contiguous()  # [out, in]
        self.bias = None if bias is None else bias.to(env.device, torch.float32).contiguous()
        self.n_out, self.n_in = self.weight.shape

    def __call__(self, a: torch.Tensor, ctx: StepContext, *, activation: str = "none", residual: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None, final: bool = False) -> torch.Tensor:
        """``final``: the caller does not touch ``residual`` again in its ``forward``. Where the block allows it
        (``ctx.may_defer``) the product may then leave the sum of its K ranges to the norm that follows."""
        if ctx.pending is not None:
            ctx.settle()  # the unfinished product's ranges live in the workspace that this one is about to use
        if out is None:
            out = residual if residual is not None else ctx.empty(a.shape[0], self.n_out, out_dtype)
        if final and ctx.may_defer and residual is out:
            ctx.pending = ctx.kernels.linear(a, self.weight, self.bias, out, activation=activation, residual=residual, may_leave_pending=True)
        else:
            ctx.kernels.linear(a, self.weight, self.bias, out, activation=activation, residual=residual)
        return out
