"""The description of a model as data: what ``models/<architecture>.py`` produces from a
configuration and what ``parts.decoder`` builds a runnable model from.

A part (norm, position encoding, mixer, feed-forward, embedding, head) is described by its
family, its kind (a name in that family's registry), its sizes and constants, and the
checkpoint tensor behind each of its parameters. A layer names the block that arranges its
parts and the parts themselves by the role they play in that block: which roles there are is
the block's business (the pre-norm block has ``norm1``, ``mixer``, ``norm2``,
``feed_forward``; a block with parallel branches, four norms or no feed-forward names others).
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
    family: str = ""
    """The registry the kind is looked up in: "norm", "mixer", "feed_forward", "position", "embedding" or "head".
    Empty: the one registry that knows the kind."""


class LayerSpec:
    """``block``: the kind of block; ``parts``: role in that block -> part. Roles read and write like attributes
    (``layer.mixer``, ``layer.norm1 = ...``)."""

    def __init__(self, block: str, parts: Optional[Dict[str, PartSpec]] = None, **roles: PartSpec):
        object.__setattr__(self, "block", block)
        object.__setattr__(self, "parts", {**(parts or {}), **roles})

    def __getattr__(self, role: str) -> PartSpec:
        try:
            return object.__getattribute__(self, "parts")[role]
        except KeyError:
            raise AttributeError(f"this layer ({self.block}) has no part {role!r}; it has {', '.join(self.parts)}") from None

    def __setattr__(self, role: str, value) -> None:
        if role == "block":
            object.__setattr__(self, role, value)
        else:
            self.parts[role] = value

    def __repr__(self) -> str:
        return f"LayerSpec({self.block!r}, {self.parts!r})"


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
    """family "embedding"; kind "token_embedding": params {position: PartSpec of a position encoding}."""
    layers: List[LayerSpec]
    plan: List[PlanEntry]
    final_norm: PartSpec
    head: PartSpec
    """family "head"; kind "tied_head" (uses the embedding's table) or "linear_head"."""
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
            for part in layer.parts.values():
                add(part)
        add(self.final_norm)
        add(self.head)
        return out
