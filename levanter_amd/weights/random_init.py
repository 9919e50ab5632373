"""Random weights from a configuration and a seed, and a model folder written from them.

The reference draws a fresh model with ``model_type.init(Vocab, config, key)``
(src/levanter/models/lm_model.py:149-150, gpt2.py:337-343). Here every tensor of the model
description is drawn from a seeded generator in the fixed order of the description: matrices,
tables and biases N(0, std), norm weights 1 + N(0, std), integer tables uniform. The draw of a
tensor depends on the seed and its name only, so a description with fewer layers is a prefix.
"""
from __future__ import annotations

import os
import zlib
from typing import Dict

import torch

from levanter_amd.config.lm_config import LmConfig
from levanter_amd.parts.spec import ModelSpec
from .safetensors_io import save_file


def random_tensors(spec: ModelSpec, seed: int, dtype: torch.dtype = torch.float32,
                   device: str | torch.device = "cpu") -> Dict[str, torch.Tensor]:
    """Draw every tensor of ``spec``. Real tensors are drawn in float32 on ``device`` and stored as ``dtype``."""
    out: Dict[str, torch.Tensor] = {}
    dev = torch.device(device)
    for name, ts in spec.all_tensors().items():
        g = torch.Generator(device=dev)
        g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (2**63 - 1))
        if ts.kind == "int":
            out[name] = torch.randint(0, 1 << 15, ts.shape, generator=g, device=dev, dtype=torch.int32)
            continue
        t = torch.empty(ts.shape, device=dev, dtype=torch.float32).normal_(0.0, spec.init_std, generator=g)
        if ts.init == "one_plus_normal":
            t += 1.0
        out[name] = t.to(dtype)
    return out


def write_random_model(config: LmConfig, seed: int, model_dir: str, dtype: torch.dtype = torch.float32) -> str:
    """Write ``config.json`` and ``model.safetensors`` of a randomly initialised model; returns the folder."""
    os.makedirs(model_dir, exist_ok=True)
    config.save(model_dir)
    tensors = random_tensors(config.model_spec(), seed, dtype=dtype, device="cpu")
    save_file(tensors, os.path.join(model_dir, "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return model_dir
