"""Registries of part kinds. Each family (norm, position encoding, mixer, feed-forward, block,
head) maps a kind name to a class; a model description names kinds, ``build_part`` constructs
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
