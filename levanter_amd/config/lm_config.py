"""The registry from an architecture's name to its configuration class, and the base class.

The reference keeps a plugin registry on ``LmConfig`` (src/levanter/models/lm_model.py:114-150)
that maps a name such as ``"gpt2"`` to a config class, and each config class knows its model
(``model_type``, src/levanter/models/gpt2.py:74-76) and how to read a checkpoint's
``config.json`` (``from_hf_config``, gpt2.py:102-117). Here the registry key is the
``model_type`` field of ``config.json``.
"""
from __future__ import annotations

import json
import os
from typing import Any, ClassVar, Dict, Type


class ConfigError(ValueError):
    """A configuration that cannot be used: unknown architecture, bad or missing key."""


class LmConfig:
    """Base of all model configurations. Subclasses are dataclasses whose fields carry the
    architecture's own ``config.json`` key names."""

    _registry: ClassVar[Dict[str, Type["LmConfig"]]] = {}
    model_type_name: ClassVar[str] = ""

    # ---- registry -------------------------------------------------------------
    @classmethod
    def register_subclass(cls, name: str):
        """Class decorator: ``@LmConfig.register_subclass("gpt2")`` (lm_model.py:115, gpt2.py:34)."""

        def deco(sub: Type["LmConfig"]) -> Type["LmConfig"]:
            if name in cls._registry and cls._registry[name] is not sub:
                raise ConfigError(f"architecture name {name!r} is already registered to {cls._registry[name].__name__}")
            sub.model_type_name = name
            cls._registry[name] = sub
            return sub

        return deco

    @classmethod
    def unregister(cls, name: str) -> None:
        cls._registry.pop(name, None)

    @classmethod
    def get_choice_class(cls, name: str) -> Type["LmConfig"]:
        _discover()
        try:
            return cls._registry[name]
        except KeyError:
            known = ", ".join(sorted(cls._registry)) or "(none)"
            raise ConfigError(f"unknown model_type {name!r}; registered architectures: {known}") from None

    @classmethod
    def known_architectures(cls):
        _discover()
        return sorted(cls._registry)

    # ---- reading config.json --------------------------------------------------
    @classmethod
    def from_hf_config(cls, hf_config: Dict[str, Any]) -> "LmConfig":
        raise NotImplementedError

    def to_hf_config(self) -> Dict[str, Any]:
        raise NotImplementedError

    def model_spec(self):
        """The description of the model (layers, their parts, the order they run in, the
        checkpoint tensor each parameter comes from) that ``parts.decoder`` builds."""
        raise NotImplementedError

    @staticmethod
    def load(model_dir: str) -> "LmConfig":
        """Read ``config.json`` of a model folder and build the registered configuration."""
        path = os.path.join(model_dir, "config.json")
        if not os.path.isfile(path):
            raise ConfigError(f"no config.json in {model_dir!r}")
        with open(path) as f:
            raw = json.load(f)
        return LmConfig.from_dict(raw)

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "LmConfig":
        if "model_type" not in raw:
            raise ConfigError("config.json has no 'model_type' key")
        return LmConfig.get_choice_class(raw["model_type"]).from_hf_config(raw)

    def save(self, model_dir: str) -> None:
        os.makedirs(model_dir, exist_ok=True)
        with open(os.path.join(model_dir, "config.json"), "w") as f:
            json.dump(self.to_hf_config(), f, indent=2)


_discovered = False


def _discover() -> None:
    """Import the architectures that ship with the package (the reference auto-discovers
    ``levanter.models``, lm_model.py:115)."""
    global _discovered
    if not _discovered:
        _discovered = True
        import levanter_amd.models  # noqa: F401
