"""The description of a model as data: what ``models/<architecture>.py`` produces from a
configuration and what ``parts.decoder`` builds a runnable model from.

A part (norm, position encoding, mixer, feed-forward) is described by its kind (a name in
that part family's registry), its sizes and constants, and the checkpoint tensor behind each
of its parameters. A layer names one part of each family and the block that arranges them.
The order in which layers run is a list of ``PlanEntry``: it may name a layer twice, and an
entry may read the cache that another entry writes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class TensorSpec:
    """A checkpoint tensor a parameter is read from."""

    name: str
    shape: Tuple[int, ...]
    kind: str = "float"  # "float": a real-valued tensor; "int": an integer table, kept as int32
    init: str = "normal"  # random-weights mode: "normal" = N(0, std), "one_plus_normal" = 1 + N(0, std)


@dataclass
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, TensorSpec] = field(default_factory=dict)


@dataclass
class LayerSpec:
    block: str
    norm1: PartSpec
    mixer: PartSpec
    norm2: PartSpec
    feed_forward: PartSpec


@dataclass(frozen=True)
class PlanEntry:
    layer: int
    """Index into ``ModelSpec.layers``: whose weights run."""
    cache: int
    """Cache unit this entry's mixer reads. Entries with ``writes_cache`` own their unit."""
    writes_cache: bool = True
    """False: the mixer only reads the unit, which an earlier entry has written in this step."""


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    dim: int
    embedding: PartSpec
    """kind "token_embedding": params {position: PartSpec of a position encoding}."""
    layers: List[LayerSpec]
    plan: List[PlanEntry]
    final_norm: PartSpec
    head: PartSpec
    """kind "tied_head" (reads the token table) or "linear_head"."""
    max_positions: Optional[int] = None
    """Largest sequence length the architecture itself allows (a position table's rows)."""
    strip_prefixes: Tuple[str, ...] = ()
    """Checkpoint name prefixes that may stand before every tensor name and are dropped."""
    ignored_tensors: Tuple[str, ...] = ()
    """Regular expressions of checkpoint tensors that are not parameters (masks and other buffers)."""
    stored_copies: Dict[str, str] = field(default_factory=dict)
    """Checkpoint tensors that may be present as a second copy of a parameter (a stored tied head): name -> the tensor
    it must equal. A copy that differs is an error: the model would not compute what the file's author computed."""
    init_std: float = 0.02

    def all_tensors(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}

        def add(part: PartSpec):
            for t in part.tensors.values():
                prev = out.get(t.name)
                if prev is not None and prev != t:
                    raise ValueError(f"tensor {t.name} is described twice with different shapes")
                out[t.name] = t
            for v in part.params.values():
                if isinstance(v, PartSpec):
                    add(v)

        add(self.embedding)
        for layer in self.layers:
            for part in (layer.norm1, layer.mixer, layer.norm2, layer.feed_forward):
                add(part)
        add(self.final_norm)
        add(self.head)
        return out
