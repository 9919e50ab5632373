"""Feed-forwards. Dense two-matrix unit: down(act(up(h))) (src/levanter/models/gpt2.py:150-155);
the activation runs in 32-bit inside the first product's epilogue, the residual sum in the second's."""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.kernels.library import ACTIVATIONS
from .base import BuildEnv, FeedForward, StepContext
from .linear import Linear
from .registry import FEED_FORWARDS
from .spec import PartSpec


@FEED_FORWARDS.register("dense_mlp")
class DenseMlp(FeedForward):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.activation = p["activation"]
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"dense_mlp: unknown activation {self.activation!r}")
        layout = p.get("weight_layout", "out_in")
        self.up = Linear(tensors["up.weight"], tensors.get("up.bias"), layout, env)
        self.down = Linear(tensors["down.weight"], tensors.get("down.bias"), layout, env)
        if (self.up.n_in, self.up.n_out) != (p["dim"], p["inner_dim"]) or (self.down.n_in, self.down.n_out) != (p["inner_dim"], p["dim"]):
            raise ValueError("dense_mlp: weights do not have the sizes of the description")

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        m = self.up(h, ctx, activation=self.activation)
        self.down(m, ctx, residual=x, final=True)
