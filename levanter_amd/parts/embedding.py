"""Embeddings: from token ids to the residual stream's first value. GPT-2: the token's row plus the row of its
absolute position (src/levanter/models/gpt2.py:291-308), summed in 32-bit by one kernel."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, Embedding, StepContext
from .registry import EMBEDDINGS, part_class
from .spec import PartSpec


def nested_tensors(spec: PartSpec, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The loaded tensors of a part under its local names. The tensors of a part nested in its parameters (an
    embedding's position encoding, an attention's rotation) travel along as ``<parameter>.<local name>``."""
    out = {local: tensors[ts.name] for local, ts in spec.tensors.items()}
    for param, v in spec.params.items():
        if isinstance(v, PartSpec):
            out.update({f"{param}.{k}": t for k, t in nested_tensors(v, tensors).items()})
    return out


def tensors_of_nested(param: str, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """What ``nested_tensors`` carried along for the part in parameter ``param``, under that part's local names."""
    prefix = param + "."
    return {k[len(prefix):]: t for k, t in tensors.items() if k.startswith(prefix)}


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Embedding):
    """params: ``vocab_size``, ``dim``, ``position`` (the description of a position encoding, or None); tensor ``table``."""

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.vocab_size = int(spec.params["vocab_size"])
        self.dim = int(spec.params["dim"])
        self.table = tensors["table"].to(env.device, env.dtype).contiguous()
        pos_spec: Optional[PartSpec] = spec.params.get("position")
        self.position = None
        if pos_spec is not None:
            self.position = part_class(pos_spec.kind, pos_spec.family or "position")(pos_spec, tensors_of_nested("position", tensors), env)

    @property
    def graph_safe(self) -> bool:
        return self.position is None or bool(self.position.graph_safe)

    @property
    def max_positions(self) -> Optional[int]:
        return None if self.position is None else self.position.max_positions

    def __call__(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.empty(ctx.n_tokens, self.dim, torch.float32)
        pos_table = None if self.position is None else self.position.embedding_table()
        ctx.kernels.embed(ctx.tokens, ctx.attention.positions, self.table, pos_table, x)
        return x
