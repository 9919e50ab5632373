"""Weights by checkpoint tensor name, checked against the model description.

The reference fills a shape-only template of the model from a state dict by key
(src/levanter/compat/hf_checkpoints.py:609-701), dropping an optional ``transformer.`` prefix
(hf_checkpoints.py:651-656, gpt2.py:80) and casting while it reads (:1239-1244). Here the
template is ``ModelSpec.all_tensors()``: every tensor it names must be there with its shape;
tensors it does not name are an error unless the description lists them as ignorable. All
faults of a checkpoint are reported in one error.

Real-valued tensors keep the precision they are stored in when that is bfloat16 or float32
(float16 and float64 are brought to float32); integer tables become int32. The parts cast what
they multiply with to the compute dtype when they are built.
"""
from __future__ import annotations

import re
from typing import Dict, List

import torch

from levanter_amd.parts.spec import ModelSpec
from .safetensors_io import SafetensorsError, open_model_files


class WeightsError(ValueError):
    """A checkpoint that does not fit the model: lists missing, unexpected and misshapen tensors."""

    def __init__(self, model_dir: str, missing: List[str], unexpected: List[str], wrong_shape: List[str], wrong_kind: List[str],
                 differing_copies: List[str] = ()):
        self.missing, self.unexpected, self.wrong_shape, self.wrong_kind = missing, unexpected, wrong_shape, wrong_kind
        self.differing_copies = list(differing_copies)
        lines = [f"checkpoint in {model_dir!r} does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if wrong_kind:
            lines.append(f"  wrong dtypes ({len(wrong_kind)}): " + "; ".join(wrong_kind))
        if differing_copies:
            lines.append(f"  stored copies that differ from their tensor ({len(differing_copies)}): " + "; ".join(differing_copies))
        super().__init__("\n".join(lines))


def _strip(name: str, prefixes) -> str:
    for p in prefixes:
        if name.startswith(p):
            return name[len(p):]
    return name


def load_tensors(model_dir: str, spec: ModelSpec, device: str | torch.device = "cpu") -> Dict[str, torch.Tensor]:
    """Read every tensor the description names from the folder's safetensors files."""
    files = open_model_files(model_dir)
    try:
        where: Dict[str, tuple] = {}
        for f in files:
            for key in f.keys():
                where[_strip(key, spec.strip_prefixes)] = (f, key)
        expected = spec.all_tensors()
        ignored = [re.compile(p) for p in spec.ignored_tensors]
        missing = [n for n in expected if n not in where]
        copies = {n: of for n, of in spec.stored_copies.items() if n in where}
        unexpected = [n for n in where if n not in expected and n not in copies and not any(r.fullmatch(n) for r in ignored)]
        wrong_shape, wrong_kind = [], []
        for n, ts in expected.items():
            if n not in where:
                continue
            f, key = where[n]
            dtype, shape = f.info(key)
            if tuple(shape) != tuple(ts.shape):
                wrong_shape.append(f"{n}: file has {list(shape)}, the configuration needs {list(ts.shape)}")
            is_float = dtype.is_floating_point
            if (ts.kind == "float") != is_float:
                wrong_kind.append(f"{n}: file has {dtype}, the model needs a{'n integer' if ts.kind == 'int' else ' real'} tensor")
        differing = []
        for n, of in copies.items():  # e.g. the stored head of a model whose head is its token table
            if of not in where:
                continue
            (f, key), (f0, key0) = where[n], where[of]
            if f.info(key)[1] != f0.info(key0)[1]:
                differing.append(f"{n}: file has {list(f.info(key)[1])}, {of} has {list(f0.info(key0)[1])}")
            elif not torch.equal(f.tensor(key).float(), f0.tensor(key0).float()):
                differing.append(f"{n} is not equal to {of} (the model uses {of} for both)")
        if missing or unexpected or wrong_shape or wrong_kind or differing:
            raise WeightsError(model_dir, sorted(missing), sorted(unexpected), wrong_shape, wrong_kind, differing)
        out: Dict[str, torch.Tensor] = {}
        for n, ts in expected.items():
            f, key = where[n]
            t = f.tensor(key)
            if ts.kind == "int":
                t = t.to(torch.int32)
            elif t.dtype not in (torch.bfloat16, torch.float32):
                t = t.to(torch.float32)
            out[n] = t.to(device) if str(device) != "cpu" else t.clone()
        return out
    finally:
        for f in files:
            f.close()


__all__ = ["WeightsError", "SafetensorsError", "load_tensors"]
