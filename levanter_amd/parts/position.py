"""Position encodings. GPT-2 adds a learned row per absolute position to the token embedding
(src/levanter/models/gpt2.py:291-296,302-308) and has nothing inside attention."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, PositionEncoding
from .registry import POSITION_ENCODINGS
from .spec import PartSpec


@POSITION_ENCODINGS.register("learned_absolute")
class LearnedAbsolutePosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        self.max_positions = int(spec.params["n_positions"])
        self.table = tensors["table"].to(env.device, env.dtype).contiguous()

    def embedding_table(self) -> Optional[torch.Tensor]:
        return self.table


@POSITION_ENCODINGS.register("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
