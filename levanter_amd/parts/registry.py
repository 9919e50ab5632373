"""Registries of part kinds. Each family (norm, position encoding, mixer, feed-forward, embedding,
head, block) maps a kind name to a class; a model description names kinds, ``build_part`` constructs
them. Registering a new kind needs no change to the framework's files:

    @MIXERS.register("my_mixer")
    class MyMixer(Mixer): ...
"""
from __future__ import annotations

from typing import Callable, Dict, Generic, Type, TypeVar

T = TypeVar("T")


class PartRegistry(Generic[T]):
    def __init__(self, family: str):
        self.family = family
        self._kinds: Dict[str, Type[T]] = {}

    def register(self, kind: str) -> Callable[[Type[T]], Type[T]]:
        def deco(cls: Type[T]) -> Type[T]:
            if kind in self._kinds and self._kinds[kind] is not cls:
                raise ValueError(f"{self.family} kind {kind!r} is already registered to {self._kinds[kind].__name__}")
            self._kinds[kind] = cls
            cls.kind = kind
            return cls

        return deco

    def unregister(self, kind: str) -> None:
        self._kinds.pop(kind, None)

    def get(self, kind: str) -> Type[T]:
        try:
            return self._kinds[kind]
        except KeyError:
            known = ", ".join(sorted(self._kinds)) or "(none)"
            raise KeyError(f"unknown {self.family} kind {kind!r}; registered: {known}") from None

    def kinds(self):
        return sorted(self._kinds)


NORMS: PartRegistry = PartRegistry("norm")
POSITION_ENCODINGS: PartRegistry = PartRegistry("position encoding")
MIXERS: PartRegistry = PartRegistry("mixer")
FEED_FORWARDS: PartRegistry = PartRegistry("feed-forward")
BLOCKS: PartRegistry = PartRegistry("block")
HEADS: PartRegistry = PartRegistry("head")
EMBEDDINGS: PartRegistry = PartRegistry("embedding")

FAMILIES: Dict[str, PartRegistry] = {"norm": NORMS, "position": POSITION_ENCODINGS, "mixer": MIXERS, "feed_forward": FEED_FORWARDS,
                                     "embedding": EMBEDDINGS, "head": HEADS}


def part_class(kind: str, family: str = ""):
    """The class of a part: from its family's registry, or (no family given) from the one registry that knows the kind."""
    if family:
        try:
            return FAMILIES[family].get(kind)
        except KeyError as e:
            if family not in FAMILIES:
                raise KeyError(f"unknown part family {family!r}; families: {', '.join(FAMILIES)}") from None
            raise e
    found = [(name, reg) for name, reg in FAMILIES.items() if kind in reg._kinds]
    if len(found) == 1:
        return found[0][1].get(kind)
    if not found:
        raise KeyError(f"no part family has a kind {kind!r}")
    raise KeyError(f"the kind {kind!r} exists in several families ({', '.join(n for n, _ in found)}); name the family in the description")
