"""Configuration from a YAML file plus dotted command-line overrides.

The reference wraps its entry points with ``levanter.config.main``, which parses a dataclass
from ``--config_path file.yaml`` and overrides of the form ``--a.b.c value`` with draccus
(src/levanter/config.py:79-169). This is the same surface for plain (nested) dataclasses.
"""
from __future__ import annotations

import dataclasses
import sys
import typing
from typing import Any, Dict, List, Optional, Sequence, Type, TypeVar

import yaml

from .lm_config import ConfigError

T = TypeVar("T")


def _set_dotted(d: Dict[str, Any], dotted: str, value: Any) -> None:
    keys = dotted.split(".")
    for k in keys[:-1]:
        d = d.setdefault(k, {})
        if not isinstance(d, dict):
            raise ConfigError(f"--{dotted}: {k!r} is not a section")
    d[keys[-1]] = value


def parse_overrides(argv: Sequence[str]) -> Dict[str, Any]:
    """``--a.b value`` / ``--a.b=value`` pairs into a nested dict; values are read as YAML scalars or lists."""
    out: Dict[str, Any] = {}
    i = 0
    argv = list(argv)
    while i < len(argv):
        arg = argv[i]
        if not arg.startswith("--"):
            raise ConfigError(f"unexpected argument {arg!r}; options look like --name value or --section.name value")
        name = arg[2:]
        if "=" in name:
            name, raw = name.split("=", 1)
            i += 1
        else:
            vals: List[str] = []
            i += 1
            while i < len(argv) and not argv[i].startswith("--"):
                vals.append(argv[i])
                i += 1
            raw = "true" if not vals else (vals[0] if len(vals) == 1 else None)
            if raw is None:
                _set_dotted(out, name, [yaml.safe_load(v) for v in vals])
                continue
        _set_dotted(out, name, yaml.safe_load(raw))
    return out


def _merge(base: Dict[str, Any], over: Dict[str, Any]) -> Dict[str, Any]:
    out = dict(base)
    for k, v in over.items():
        out[k] = _merge(out[k], v) if isinstance(v, dict) and isinstance(out.get(k), dict) else v
    return out


def from_dict(cls: Type[T], data: Dict[str, Any], path: str = "") -> T:
    """Build dataclass ``cls`` from a nested dict; unknown keys are an error that lists the known ones."""
    if not dataclasses.is_dataclass(cls):
        raise TypeError(f"{cls} is not a dataclass")
    hints = typing.get_type_hints(cls)
    fields = {f.name: f for f in dataclasses.fields(cls) if f.init}
    unknown = [k for k in data if k not in fields]
    if unknown:
        raise ConfigError(f"unknown option(s) {', '.join(path + k for k in unknown)}; known: {', '.join(path + k for k in fields)}")
    kwargs = {}
    for name, value in data.items():
        t = hints.get(name)
        origin = typing.get_origin(t)
        args = [a for a in typing.get_args(t) if a is not type(None)] if origin is typing.Union else []
        target = t if dataclasses.is_dataclass(t) else next((a for a in args if dataclasses.is_dataclass(a)), None)
        if target is not None and isinstance(value, dict):
            value = from_dict(target, value, path + name + ".")
        kwargs[name] = value
    try:
        return cls(**kwargs)
    except TypeError as e:
        raise ConfigError(f"{path or cls.__name__}: {e}") from None


def describe_options(cls: Type, prefix: str = "") -> List[str]:
    """One line per option of dataclass ``cls`` (sections as dotted names) with its type and default."""
    lines: List[str] = []
    hints = typing.get_type_hints(cls)
    for f in dataclasses.fields(cls):
        if not f.init:
            continue
        t = hints.get(f.name)
        args = [a for a in typing.get_args(t) if a is not type(None)] if typing.get_origin(t) is typing.Union else []
        target = t if dataclasses.is_dataclass(t) else next((a for a in args if dataclasses.is_dataclass(a)), None)
        if target is not None:
            lines += describe_options(target, prefix + f.name + ".")
            continue
        if f.default is not dataclasses.MISSING:
            default = repr(f.default)
        elif f.default_factory is not dataclasses.MISSING:  # type: ignore[misc]
            default = repr(f.default_factory())  # type: ignore[misc]
        else:
            default = "required"
        name = str(t).replace("typing.", "") if typing.get_origin(t) is not None else getattr(t, "__name__", str(t))
        lines.append(f"  --{prefix}{f.name} ({name}; default {default})")
    return lines


def parse_config(cls: Type[T], argv: Optional[Sequence[str]] = None) -> T:
    """``--config_path file.yaml`` (optional) plus overrides, into ``cls``. ``--help`` prints the options and exits."""
    argv = list(sys.argv[1:] if argv is None else argv)
    if any(a in ("--help", "-h") for a in argv):
        doc = (sys.modules[cls.__module__].__doc__ or "").strip()
        print((doc + "\n\n" if doc else "") + "options (also as keys of the --config_path YAML file, sections nested):\n"
              + "\n".join(describe_options(cls)))
        raise SystemExit(0)
    over = parse_overrides(argv)
    base: Dict[str, Any] = {}
    path = over.pop("config_path", None) or over.pop("config", None)
    if path is not None:
        with open(path) as f:
            base = yaml.safe_load(f) or {}
        if not isinstance(base, dict):
            raise ConfigError(f"{path}: a configuration file holds a mapping")
    return from_dict(cls, _merge(base, over))
